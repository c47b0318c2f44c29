"""StableHLO walker: the literal (unfused) path and the recognizer's host.

`Interpreter.run_block` walks a block's ops over an SSA environment and calls
`REGISTRY[name](interp, op, ins, env)`; a handler returns one array or a list
(the op-handler signature of reference src/metaljax/interpreter.py:325,
:910-927).  Before an op runs, the block's rewrite plan is consulted: an op a
recognizer absorbed is skipped, a recognized root is replaced by
`emit(interp, match, env)` (reference interpreter.py:789-848, :900-908).

Arrays.  Literal ops run on the host with numpy, on `HostArray`s: the values
plus the StableHLO element type.  bf16 has no numpy dtype, so a bf16 tensor
holds float32 values that are exactly representable in bf16 and every bf16 op
rounds its float32 result once (round to nearest even), which is what a
backend that widens bf16 arithmetic to float32 computes.  4-bit integers live
in 8-bit storage and wrap to 4 bits.  This path exists to (1) evaluate a
weight's reconstruction subtree once, at pack time, and (2) run whatever a
recognizer did not claim.  The fused quantized matmul itself never runs here:
`qmm.emit` launches the HIP kernels and raises if they are unavailable.
"""

from __future__ import annotations

import numpy as np

from . import ir
from .packing import f32_to_bf16_bits

REGISTRY = {}
_SKIP = object()


def register(*names):
    def deco(fn):
        for n in names:
            REGISTRY[n] = fn
        return fn
    return deco


class UnsupportedOp(NotImplementedError):
    pass


# ------------------------------------------------------------------ arrays ---

class HostArray:
    """A host tensor: numpy storage + the StableHLO element type."""

    __slots__ = ("a", "el", "bits", "__weakref__")

    def __init__(self, a, el):
        self.a = a
        self.el = el
        self.bits = None            # bf16 only, optional: the 16-bit patterns, for callers that need the type's own bytes

    @property
    def shape(self):
        return self.a.shape

    def __repr__(self):
        return f"HostArray({self.el}{list(self.a.shape)})"


def round_bf16(x32: np.ndarray) -> np.ndarray:
    bits = f32_to_bf16_bits(np.ascontiguousarray(x32, np.float32))
    return (bits.astype(np.uint32) << 16).view(np.float32).reshape(np.shape(x32))


_INT_BITS = {"i4": 4, "ui4": 4, "i8": 8, "ui8": 8, "i16": 16, "ui16": 16, "i32": 32, "ui32": 32,
             "i64": 64, "ui64": 64}
FLOAT_ELS = ("f16", "bf16", "f32", "f64")


def is_float(el):
    return el in FLOAT_ELS


def is_signed(el):
    return el[0] == "i" and el != "i1"


def settle(a: np.ndarray, el: str) -> HostArray:
    """Bring a freshly computed array to the storage convention of `el`."""
    dt = ir.np_dtype(el)
    if el == "bf16":
        return HostArray(round_bf16(np.asarray(a, np.float32)), el)
    if el in ("i4", "ui4"):
        a = np.asarray(a).astype(np.int64) & 15
        if el == "i4":
            a = np.where(a >= 8, a - 16, a)
        return HostArray(a.astype(dt), el)
    return HostArray(np.asarray(a).astype(dt, copy=False), el)


def from_numpy(a, el=None) -> HostArray:
    """Wrap a numpy array (float32 values for el="bf16")."""
    a = np.asarray(a)
    if el is None:
        el = {np.dtype(np.bool_): "i1", np.dtype(np.int8): "i8", np.dtype(np.uint8): "ui8",
              np.dtype(np.int16): "i16", np.dtype(np.uint16): "ui16", np.dtype(np.int32): "i32",
              np.dtype(np.uint32): "ui32", np.dtype(np.int64): "i64", np.dtype(np.uint64): "ui64",
              np.dtype(np.float16): "f16", np.dtype(np.float32): "f32",
              np.dtype(np.float64): "f64"}[a.dtype]
    return settle(a, el)


# Host copies of device tensors, one per tensor object while it lives and is
# not written: a program argument that several literal ops (or several pack
# builds) read is copied back once.  An entry holds the tensor's version
# counter, which torch bumps on every in-place write (through any view), so a
# caller that refills a buffer between calls gets a fresh copy.  (Writes torch
# cannot see -- a kernel handed the raw pointer -- would go unnoticed: the
# fused calls here only ever write into tensors they have just allocated.)
_MIRRORS = {}
MIRROR_MAX_BYTES = 16 << 20     # larger tensors (weights) are copied back whenever read: no second copy is kept
HOST_COPIES = [0]               # device -> host copies made (tests count them)


def _version(v):
    try:
        return v._version
    except RuntimeError:            # an inference-mode tensor keeps no counter: never mirrored
        return None


def _mirror_get(v):
    hit = _MIRRORS.get(id(v))
    if hit is not None and hit[0]() is v and hit[2] == _version(v):
        return hit[1]
    return None


def _mirror_put(v, h):
    import weakref
    key, version = id(v), _version(v)
    if version is not None:
        _MIRRORS[key] = (weakref.ref(v, lambda _, key=key: _MIRRORS.pop(key, None)), h, version)


def host(v) -> HostArray:
    """Any runtime value as a HostArray (device tensors are copied back)."""
    if isinstance(v, HostArray):
        return v
    if hasattr(v, "type_enum") and hasattr(v, "data"):      # an engine buffer
        return host(v.data)
    import torch
    if isinstance(v, torch.Tensor):
        hit = _mirror_get(v)
        if hit is not None:
            return hit
        if v.is_cuda:
            HOST_COPIES[0] += 1
        if v.dtype == torch.bfloat16:
            h = HostArray(v.float().cpu().numpy(), "bf16")
        else:
            h = from_numpy(v.cpu().numpy())
        if v.is_cuda and v.numel() * v.element_size() <= MIRROR_MAX_BYTES:
            _mirror_put(v, h)
        return h
    return from_numpy(v)


def _compute(el):
    """dtype the arithmetic of an element type runs in."""
    if el in ("bf16", "f16"):
        return np.float32
    return ir.np_dtype(el)


# ------------------------------------------------------------ interpreter ----

class Interpreter:
    def __init__(self, module):
        self.module = ir.parse_module(module) if isinstance(module, str) else module
        self.main = self.module.main
        self.donated_args = {i for i, a in enumerate(self.main.arg_attrs)
                             if "tf.aliasing_output" in a or a.get("jax.buffer_donor")}
        self._qmm = None            # recognizer state (metaljax_amd.qmm.State)
        self._plans = {}

    def _main_block(self):
        return self.main.body

    def invalidate_plans(self):
        self._plans = {}

    # -- rewrite plan: op -> _SKIP | (emit, match)
    def _rewrite_plan(self, block):
        plan = self._plans.get(block)
        if plan is not None:
            return plan
        plan = {}
        st = self._qmm
        if st is not None and st.active:
            from . import qmm
            for op in block.ops:
                key = op.results[0] if op.results else None
                if key is None:
                    continue
                m = st.roots.get(key)
                if m is not None:
                    plan[op] = (qmm.emit, m, qmm.emit_reads(m))
                elif key in st.skip:
                    plan[op] = _SKIP
        self._plans[block] = plan
        return plan

    def run_block(self, block, env):
        plan = self._rewrite_plan(block)
        for op in block.ops:
            if op.name == "return":
                return [env[v] for v in op.operands]
            entry = plan.get(op)
            if entry is _SKIP:
                continue                       # absorbed into a fused root: never runs
            if entry is not None:
                fuse, match, _ = entry
                out = fuse(self, match, env)
            else:
                handler = REGISTRY.get(op.name)
                if handler is None:
                    raise UnsupportedOp(f"no handler for {op.name}")
                out = handler(self, op, [env[v] for v in op.operands], env)
            if not isinstance(out, (list, tuple)):
                out = [out]
            for r, v in zip(op.results, out):
                env[r] = v
        raise RuntimeError("block has no terminator")

    def run(self, args):
        """Run @main on `args` (HostArrays, numpy arrays or device tensors)."""
        if len(args) != len(self.main.body.args):
            raise ValueError(f"@main takes {len(self.main.body.args)} arguments, got {len(args)}")
        env = dict(zip(self.main.body.args, args))
        return self.run_block(self.main.body, env)


# ---------------------------------------------------------------- handlers ---

def _ty(op, i=0):
    return op.results[i].type


@register("stablehlo.constant")
def _constant(interp, op, ins, env):
    ty = _ty(op)
    return HostArray(ir.dense_to_np(op.attrs["value"], ty), ty.el)


@register("stablehlo.iota")
def _iota(interp, op, ins, env):
    ty = _ty(op)
    d = op.attrs["iota_dimension"]
    shape = [1] * len(ty.shape)
    shape[d] = ty.shape[d]
    a = np.broadcast_to(np.arange(ty.shape[d]).reshape(shape), ty.shape)
    return settle(a, ty.el)


def _binary(fn, int_fn=None):
    def handler(interp, op, ins, env):
        a, b = host(ins[0]), host(ins[1])
        el = _ty(op).el
        ct = _compute(el)
        f = int_fn if (int_fn is not None and not is_float(el)) else fn
        with np.errstate(all="ignore"):
            return settle(f(a.a.astype(ct, copy=False), b.a.astype(ct, copy=False)), el)
    return handler


def _int_divide(a, b):
    q = np.where(b == 0, -1, np.trunc(np.divide(a, np.where(b == 0, 1, b), dtype=np.float64)))
    return q.astype(a.dtype)


REGISTRY.update({
    "stablehlo.add": _binary(np.add),
    "stablehlo.subtract": _binary(np.subtract),
    "stablehlo.multiply": _binary(np.multiply),
    "stablehlo.divide": _binary(np.divide, _int_divide),
    "stablehlo.maximum": _binary(np.maximum),
    "stablehlo.minimum": _binary(np.minimum),
    "stablehlo.power": _binary(np.power),
    "stablehlo.and": _binary(np.bitwise_and),
    "stablehlo.or": _binary(np.bitwise_or),
    "stablehlo.xor": _binary(np.bitwise_xor),
})


def _shift(kind):
    def handler(interp, op, ins, env):
        a, b = host(ins[0]), host(ins[1])
        el = _ty(op).el
        bits = _INT_BITS[el]
        av = a.a.astype(np.int64)
        sh = b.a.astype(np.int64)
        big = (sh < 0) | (sh >= bits)              # XLA: shifting past the width
        s = np.where(big, 0, sh)
        if kind == "left":
            r = np.where(big, 0, av << s)
        elif kind == "logical":
            r = np.where(big, 0, (av & ((1 << bits) - 1)) >> s)
        else:
            r = np.where(big, np.where(av < 0, -1, 0), av >> s)
        if el in ("i4", "ui4"):
            return settle(r, el)
        mask = (1 << bits) - 1
        r = r & mask
        if is_signed(el):
            r = np.where(r >= (1 << (bits - 1)), r - (1 << bits), r)
        return settle(r, el)
    return handler


REGISTRY["stablehlo.shift_left"] = _shift("left")
REGISTRY["stablehlo.shift_right_logical"] = _shift("logical")
REGISTRY["stablehlo.shift_right_arithmetic"] = _shift("arithmetic")


def _unary(fn):
    def handler(interp, op, ins, env):
        a = host(ins[0])
        el = _ty(op).el
        with np.errstate(all="ignore"):
            return settle(fn(a.a.astype(_compute(el), copy=False)), el)
    return handler


REGISTRY.update({
    "stablehlo.negate": _unary(np.negative),
    "stablehlo.abs": _unary(np.abs),
    "stablehlo.exponential": _unary(np.exp),
    "stablehlo.log": _unary(np.log),
    "stablehlo.sqrt": _unary(np.sqrt),
    "stablehlo.rsqrt": _unary(lambda x: 1.0 / np.sqrt(x)),
    "stablehlo.tanh": _unary(np.tanh),
    "stablehlo.logistic": _unary(lambda x: 1.0 / (1.0 + np.exp(-x))),
    "stablehlo.floor": _unary(np.floor),
    "stablehlo.ceil": _unary(np.ceil),
    "stablehlo.round_nearest_even": _unary(np.rint),
    "stablehlo.not": _unary(np.invert),
    "stablehlo.sign": _unary(np.sign),
})


@register("stablehlo.convert")
def _convert(interp, op, ins, env):
    a = host(ins[0])
    el = _ty(op).el
    src = a.a
    if is_float(a.el) and not is_float(el):
        if el == "i1":
            return settle(src != 0, el)
        with np.errstate(all="ignore"):
            src = np.trunc(src.astype(np.float64))
            info = np.iinfo(ir.np_dtype(el))
            src = np.clip(np.nan_to_num(src, nan=0.0), info.min, info.max)
    if el == "i1":
        return settle(src != 0, el)
    return settle(src, el)


@register("stablehlo.bitcast_convert")
def _bitcast(interp, op, ins, env):
    a = host(ins[0])
    ty = _ty(op)
    if "bf16" in (a.el, ty.el) or a.el in ("i4", "ui4") or ty.el in ("i4", "ui4"):
        if a.el == "bf16":
            bits = f32_to_bf16_bits(a.a)
            return settle(bits.view(ir.np_dtype(ty.el)).reshape(ty.shape), ty.el)
        if ty.el == "bf16" and a.a.dtype.itemsize == 2:
            f = (a.a.view(np.uint16).astype(np.uint32) << 16).view(np.float32)
            return HostArray(f.reshape(ty.shape), "bf16")
        raise UnsupportedOp(f"bitcast_convert {a.el} -> {ty.el}")
    return HostArray(np.ascontiguousarray(a.a).view(ir.np_dtype(ty.el)).reshape(ty.shape), ty.el)


@register("stablehlo.reshape")
def _reshape(interp, op, ins, env):
    a = host(ins[0])
    return HostArray(a.a.reshape(_ty(op).shape), a.el)


@register("stablehlo.transpose")
def _transpose(interp, op, ins, env):
    a = host(ins[0])
    return HostArray(np.transpose(a.a, ir.i64_list(op, "permutation")), a.el)


@register("stablehlo.broadcast_in_dim")
def _broadcast_in_dim(interp, op, ins, env):
    a = host(ins[0])
    ty = _ty(op)
    dims = ir.i64_list(op, "broadcast_dimensions")
    shape = [1] * len(ty.shape)
    for i, d in enumerate(dims):
        shape[d] = a.a.shape[i]
    return HostArray(np.broadcast_to(a.a.reshape(shape), ty.shape), a.el)


@register("stablehlo.slice")
def _slice(interp, op, ins, env):
    a = host(ins[0])
    idx = tuple(slice(s, l, t) for s, l, t in zip(op.attrs["start_indices"],
                                                  op.attrs["limit_indices"], op.attrs["strides"]))
    return HostArray(a.a[idx], a.el)


@register("stablehlo.concatenate")
def _concatenate(interp, op, ins, env):
    arrs = [host(x) for x in ins]
    d = op.attrs.get("dim", op.attrs.get("dimension"))
    return HostArray(np.concatenate([x.a for x in arrs], axis=d), arrs[0].el)


@register("stablehlo.compare")
def _compare(interp, op, ins, env):
    a, b = host(ins[0]), host(ins[1])
    fn = {"EQ": np.equal, "NE": np.not_equal, "LT": np.less, "LE": np.less_equal,
          "GT": np.greater, "GE": np.greater_equal}[op.attrs["comparison_direction"]]
    with np.errstate(all="ignore"):
        return HostArray(fn(a.a, b.a), "i1")


@register("stablehlo.select")
def _select(interp, op, ins, env):
    p, a, b = host(ins[0]), host(ins[1]), host(ins[2])
    return HostArray(np.where(p.a, a.a, b.a), a.el)


@register("stablehlo.clamp")
def _clamp(interp, op, ins, env):
    lo, x, hi = host(ins[0]), host(ins[1]), host(ins[2])
    return HostArray(np.minimum(np.maximum(x.a, lo.a), hi.a).astype(x.a.dtype), x.el)


@register("stablehlo.dynamic_slice")
def _dynamic_slice(interp, op, ins, env):
    a = host(ins[0])
    sizes = op.attrs.get("sizes", op.attrs.get("slice_sizes"))
    starts = [int(host(i).a) for i in ins[1:]]
    idx = tuple(slice(min(max(s, 0), d - n), min(max(s, 0), d - n) + n)
                for s, n, d in zip(starts, sizes, a.a.shape))
    return HostArray(a.a[idx], a.el)


@register("stablehlo.dynamic_update_slice")
def _dynamic_update_slice(interp, op, ins, env):
    a, u = host(ins[0]), host(ins[1])
    starts = [int(host(i).a) for i in ins[2:]]
    out = np.array(a.a, copy=True)
    idx = tuple(slice(min(max(s, 0), d - n), min(max(s, 0), d - n) + n)
                for s, n, d in zip(starts, u.a.shape, a.a.shape))
    out[idx] = u.a
    return HostArray(out, a.el)


@register("stablehlo.gather")
def _gather(interp, op, ins, env):
    """General gather; start indices are clamped so every slice stays in
    bounds, as XLA does (reference src/metaljax/ops/gather.py:82-181, :116)."""
    operand, idx = host(ins[0]), host(ins[1])
    dn = op.attrs["dimension_numbers"][1]
    offset_dims = dn.get("offset_dims", [])
    collapsed = dn.get("collapsed_slice_dims", [])
    batching = dn.get("operand_batching_dims", [])
    if batching:
        raise UnsupportedOp("gather with batching dims")
    start_map = dn.get("start_index_map", [])
    ivd = dn.get("index_vector_dim", idx.a.ndim - 1)
    sizes = op.attrs["slice_sizes"]
    ind = idx.a.astype(np.int64)
    if ivd == ind.ndim:
        ind = ind[..., None]
    ind = np.moveaxis(ind, ivd, -1)                    # [batch..., len(start_map)]
    bshape = ind.shape[:-1]
    src = operand.a
    full = np.zeros(bshape + (src.ndim,), np.int64)
    for j, d in enumerate(start_map):
        full[..., d] = np.clip(ind[..., j], 0, src.shape[d] - sizes[d])
    kept = [d for d in range(src.ndim) if d not in collapsed]
    # index grids: batch dims first, then the kept slice dims
    grids = []
    nb = len(bshape)
    for d in range(src.ndim):
        g = full[..., d].reshape(bshape + (1,) * len(kept))
        if d in kept:
            k = kept.index(d)
            shp = [1] * (nb + len(kept))
            shp[nb + k] = sizes[d]
            g = g + np.arange(sizes[d]).reshape(shp)
        grids.append(g)
    out = src[tuple(grids)]                            # [batch..., kept slice dims...]
    # place offset dims where the result wants them
    rank = nb + len(kept)
    batch_positions = [d for d in range(rank) if d not in offset_dims]
    perm = [0] * rank
    for i, p in enumerate(batch_positions):
        perm[p] = i
    for i, p in enumerate(offset_dims):
        perm[p] = nb + i
    out = np.transpose(out, perm)
    return HostArray(out.reshape(_ty(op).shape), operand.el)


# ---- the literal dot on the device -----------------------------------------
# A dot the recognizer left alone (or gave back) still belongs on the GPU when
# there is one, as in the reference, whose literal dot is a device matmul
# (reference src/metaljax/ops/linalg.py:91-142): operands widened to float32,
# one library matmul (float32 accumulate), one rounding to the result type.
_DEVICE_DOT_ELS = {"bf16": "bfloat16", "f16": "float16", "f32": "float32"}
_DEVICE_DOT_MIN_MACS = 1 << 22         # below this the copies cost more than the product


def _device_dot_pays(ins, lc, ty) -> bool:
    """Is there a GPU, and is the product large enough (or an operand already
    there) for the device to be the place to run it?"""
    try:
        import torch
    except ImportError:
        return False
    if not torch.cuda.is_available():
        return False
    if any(isinstance(x, torch.Tensor) and x.is_cuda for x in ins):
        return True
    a = ins[0]
    shape = tuple(a.shape) if isinstance(a, torch.Tensor) else host(a).a.shape
    k = 1
    for d in lc:
        k *= shape[d]
    return ty.size * k >= _DEVICE_DOT_MIN_MACS


def _as_device_f32(v):
    import torch
    if isinstance(v, torch.Tensor):
        return v.cuda().float()
    h = host(v)
    return torch.from_numpy(np.array(h.a, dtype=np.float32)).cuda()


def _dot_general_device(ins, lb, rb, lc, rc, ty):
    import torch
    A, B = _as_device_f32(ins[0]), _as_device_f32(ins[1])
    af = [d for d in range(A.dim()) if d not in lb and d not in lc]
    bf = [d for d in range(B.dim()) if d not in rb and d not in rc]
    A = A.permute(lb + af + lc)
    B = B.permute(rb + bf + rc)
    nb = len(lb)
    bs = tuple(A.shape[:nb])
    k = 1
    for d in A.shape[nb + len(af):]:
        k *= d
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        out = torch.matmul(A.reshape(bs + (-1, k)), B.reshape(bs + (-1, k)).transpose(-1, -2))
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
    return out.reshape(tuple(ty.shape)).to(getattr(torch, _DEVICE_DOT_ELS[ty.el]))


@register("stablehlo.dot_general")
def _dot_general(interp, op, ins, env):
    """The literal dot: operands widened to float32 (float64 for f64), product
    accumulated there, one rounding to the result type (reference
    src/metaljax/ops/linalg.py:91-142)."""
    lb, rb, lc, rc = ir.dot_dims(op)
    ty = _ty(op)
    if ty.el in _DEVICE_DOT_ELS and _device_dot_pays(ins, lc, ty):
        return _dot_general_device(ins, lb, rb, lc, rc, ty)
    a, b = host(ins[0]), host(ins[1])
    ct = np.float64 if ty.el == "f64" else (np.float32 if is_float(ty.el) else np.int64)
    A, B = a.a.astype(ct), b.a.astype(ct)
    af = [d for d in range(A.ndim) if d not in lb and d not in lc]
    bf = [d for d in range(B.ndim) if d not in rb and d not in rc]
    A = np.transpose(A, lb + af + lc)
    B = np.transpose(B, rb + bf + rc)
    nb = len(lb)
    bs = A.shape[:nb]
    k = int(np.prod(A.shape[nb + len(af):], dtype=np.int64))
    A2 = A.reshape(bs + (-1, k))
    B2 = B.reshape(bs + (-1, k))
    out = np.matmul(A2, np.swapaxes(B2, -1, -2))
    return settle(out.reshape(ty.shape), ty.el)


@register("stablehlo.reduce")
def _reduce(interp, op, ins, env):
    n = len(ins) // 2
    dims = tuple(op.attrs["dimensions"])
    body = op.attrs.get("body")
    if body is None and op.regions:
        inner = [o for o in op.regions[0].ops if o.name != "return"]
        if n == 1 and len(inner) == 1:
            body = inner[0].name
    if n != 1 or body is None:
        raise UnsupportedOp("variadic / custom reduce")
    a = host(ins[0])
    el = _ty(op).el
    fn = {"stablehlo.add": np.sum, "stablehlo.maximum": np.max, "stablehlo.minimum": np.min,
          "stablehlo.multiply": np.prod, "stablehlo.or": np.any, "stablehlo.and": np.all}.get(body)
    if fn is None:
        raise UnsupportedOp(f"reduce with {body}")
    src = a.a.astype(np.float32 if el in ("bf16", "f16") else a.a.dtype)
    return settle(fn(src, axis=dims), el)


def top_k(a: np.ndarray, k: int):
    """(values, int32 indices) of the k largest entries along the last axis,
    largest first, equal values in index order."""
    order = np.argsort(-a, axis=-1, kind="stable")[..., :k]
    return np.take_along_axis(a, order, axis=-1), order.astype(np.int32)


@register("chlo.top_k")
def _top_k(interp, op, ins, env):
    a = host(ins[0])
    k = op.attrs.get("k", op.results[0].type.shape[-1])
    vals, idx = top_k(a.a.astype(np.float32 if a.el in ("bf16", "f16") else a.a.dtype), k)
    return [settle(vals, op.results[0].type.el), settle(idx, op.results[1].type.el)]


@register("stablehlo.composite")
def _composite(interp, op, ins, env):
    """A composite runs as what it names when that is known here (a top-k
    arrives wrapped like this after a portable-artifact round trip), else as
    its decomposition."""
    if op.attrs.get("name") == "chlo.top_k":
        return _top_k(interp, op, ins, env)
    f = interp.module.funcs[str(op.attrs["decomposition"]).lstrip("@")]
    return interp.run_block(f.body, dict(zip(f.body.args, ins)))


@register("func.call")
def _call(interp, op, ins, env):
    f = interp.module.funcs[op.attrs["callee"]]
    return interp.run_block(f.body, dict(zip(f.body.args, ins)))


@register("stablehlo.while")
def _while(interp, op, ins, env):
    cond, body = op.regions
    state = list(ins)
    while True:
        cenv = dict(env)
        cenv.update(zip(cond.args, state))
        (p,) = interp.run_block(cond, cenv)
        if not bool(host(p).a):
            return state
        benv = dict(env)
        benv.update(zip(body.args, state))
        state = interp.run_block(body, benv)


def _identity(interp, op, ins, env):
    return list(ins)


REGISTRY["sdy.sharding_constraint"] = _identity
REGISTRY["stablehlo.optimization_barrier"] = _identity
