"""Expert dispatch: a dense mixture-of-experts block rewritten onto the
expert-indexed quantized product.

A model written against jax.numpy runs every expert on every token and lets
routing weights that are zero off a top-k selection null the rest:

    S   = sum_k one_hot(idx[t, k], E) * w[t, k]        idx, values = top_k(logits, K)
    out = sum_e Y[e, t, ...] * S[t, e]                 Y = expert_e(x) for EVERY e

The job, the accepted graph shape and the failure behaviour are those of the
reference's recognizer (reference src/metaljax/moe.py:335-442 router match,
:522-810 pair-space planner, :1112-1153 verification, :1283-1340 and
:1425-1461 emission); the formulation is this package's own, and it serves the
QUANTIZED case only: every per-expert dot of the region must already be a
quantized-matmul match, whose pack the dispatch then reads through
`kernels.gather_qmm` (a region with a float per-expert weight stays dense).

  * `prove_router` shows from structure alone that S is w scattered at a
    top-k's indices (the one-hot is matched down to `compare EQ(indices,
    iota over experts)`), so every entry off the selection is an exact zero.
  * `PairPlan` re-plans Y over the P = T * K selected (token, expert) pairs.
    A region value of dense shape D with its expert axis at `e` and token
    axis at `t` becomes an array `[P] + D without those axes`: per-expert data
    is gathered by the pair's expert, per-token data by its token, each
    per-expert dot becomes one expert-indexed product, everything between the
    dots runs on P rows.  Lowering appends one closure per value to a list;
    running the dispatch is running the list.
  * What does not carry the expert axis is not region work: it is computed
    once, densely, by the program itself and gathered on the way in.
  * Every dispatch is checked numerically before first use, on synthetic
    logits (`verify`): the router tail below the top-k depends on nothing but
    the logits, so S can be evaluated on random draws and compared with the
    scatter of w at idx.  METALJAX_MOE_VERIFY=0 skips it.

Anything not understood rejects the dispatch and the dense block runs as it
is.  The gathered sum adds K terms where the dense one adds E (E - K of them
exact zeros), so results differ at float32 reduction-order scale; an unrouted
expert's overflow, which the dense sum turns into NaN through 0 * inf, does
not reach the gathered result.  METALJAX_MOE=0 disables the recognizer.
"""

from __future__ import annotations

import os

import numpy as np

from . import ir
from .interpreter import REGISTRY, HostArray, host, settle
from .packing import Reject
from .recognize import OPAQUE_OPS, count, dims_of, elem, op_key

ENABLED = os.environ.get("METALJAX_MOE", "1") != "0"           # (reference moe.py:93; its tests flip it at run time)
VERIFY = os.environ.get("METALJAX_MOE_VERIFY", "1") != "0"
VERIFY_DRAWS = int(os.environ.get("METALJAX_MOE_VERIFY_DRAWS", "3"))
_DEBUG = os.environ.get("METALJAX_DEBUG", "") == "1"
# The reference's keys (moe.py:100-101; "gather_mm", its float-weight product, stays 0 here: experts
# whose weights are not quantized packs are left to the dense block) plus two of this package's own.
STATS = {"recognized": 0, "verified": 0, "fallbacks": 0, "gather_qmm": 0, "gather_mm": 0,
         "dispatches": 0, "host_copies": 0}


def stats() -> dict:
    return dict(STATS)


def reset_stats():
    for k in STATS:
        STATS[k] = 0


def _debug(text):
    if _DEBUG:
        print(f"[metaljax_amd] moe: {text}", flush=True)


# Ops that compute element i of the result from element i of same-shaped
# operands (rank-0 operands aside): they run unchanged on pair-space arrays.
_ELEMENTWISE = frozenset("""
    stablehlo.abs stablehlo.add stablehlo.and stablehlo.ceil stablehlo.clamp stablehlo.compare
    stablehlo.convert stablehlo.divide stablehlo.exponential stablehlo.floor stablehlo.log
    stablehlo.logistic stablehlo.maximum stablehlo.minimum stablehlo.multiply stablehlo.negate
    stablehlo.not stablehlo.or stablehlo.power stablehlo.round_nearest_even stablehlo.rsqrt
    stablehlo.select stablehlo.sign stablehlo.sqrt stablehlo.subtract stablehlo.tanh stablehlo.xor
""".split())


# ------------------------------------------------------- run-time pieces ----

class DevArray:
    """A device tensor plus its StableHLO element type: what a slot of a
    running dispatch holds.  Everything between the per-expert products runs
    on these, on the device (reference moe.py:1425-1461 runs its closure list
    on device arrays)."""

    __slots__ = ("t", "el")

    def __init__(self, t, el):
        self.t = t
        self.el = el


_TORCH_EL = {"i1": "bool", "i8": "int8", "i16": "int16", "i32": "int32", "i64": "int64", "ui8": "uint8",
             "f16": "float16", "bf16": "bfloat16", "f32": "float32", "f64": "float64"}
_FLOATS = ("f16", "bf16", "f32", "f64")
_WRAPPING_INTS = ("i8", "i16", "i32", "i64", "ui8")


class _HostOnly(Exception):
    """This op / element type is not modelled on the device: the fill runs on
    the host (a copy each way) instead."""


def _tdtype(el):
    import torch
    return getattr(torch, _TORCH_EL[el])


def dev(v) -> DevArray:
    """Any runtime value as a DevArray (host values are uploaded)."""
    import torch
    from . import qmm
    if isinstance(v, DevArray):
        return v
    if hasattr(v, "type_enum") and hasattr(v, "data"):
        v = v.data
    if isinstance(v, torch.Tensor):
        el = {getattr(torch, name): e for e, name in _TORCH_EL.items()}.get(v.dtype)
        if el is None:
            raise _HostOnly(str(v.dtype))
        return DevArray(qmm.to_device(v), el)
    h = host(v)
    if h.el not in _TORCH_EL:
        raise _HostOnly(h.el)
    return DevArray(qmm.to_device(h), h.el)


def _dev_elementwise(op, args, out_el):
    """One elementwise StableHLO op on device tensors, with the literal
    path's meaning: 16-bit floats are widened, computed in float32 and rounded
    once (what torch's elementwise kernels do), comparisons give i1."""
    import torch
    if out_el not in _TORCH_EL or any(a.el not in _TORCH_EL for a in args):
        raise _HostOnly(op.name)
    name = op.name[len("stablehlo."):]
    t = [a.t for a in args]
    fl = all(a.el in _FLOATS for a in args)
    binary = {"add": torch.add, "subtract": torch.sub, "multiply": torch.mul, "divide": torch.div,
              "maximum": torch.maximum, "minimum": torch.minimum, "power": torch.pow}
    unary = {"abs": torch.abs, "ceil": torch.ceil, "floor": torch.floor, "exponential": torch.exp,
             "log": torch.log, "logistic": torch.sigmoid, "negate": torch.neg, "rsqrt": torch.rsqrt,
             "sqrt": torch.sqrt, "tanh": torch.tanh, "sign": torch.sign, "round_nearest_even": torch.round}
    logic = {"and": torch.bitwise_and, "or": torch.bitwise_or, "xor": torch.bitwise_xor}
    if name in binary and fl:
        return binary[name](t[0], t[1])
    if name == "sign" and fl:
        return torch.where(torch.isnan(t[0]), t[0], torch.sign(t[0]))      # torch's sign of a NaN is 0
    if name in unary and fl:
        return unary[name](t[0])
    ints = all(a.el in _WRAPPING_INTS for a in args)
    if ints and name in ("add", "subtract", "multiply", "maximum", "minimum"):
        return binary[name](t[0], t[1])                                    # two's-complement wrap, as numpy's
    if ints and name in ("abs", "negate", "sign") and not args[0].el.startswith("ui"):
        return unary[name](t[0])
    if name in logic and not fl:
        return logic[name](t[0], t[1])
    if name == "not" and not fl:
        return torch.bitwise_not(t[0])
    if name == "compare":
        fn = {"EQ": torch.eq, "NE": torch.ne, "LT": torch.lt, "LE": torch.le, "GT": torch.gt,
              "GE": torch.ge}[op.attrs["comparison_direction"]]
        return fn(t[0], t[1])
    if name == "select":
        return torch.where(t[0], t[1], t[2])
    if name == "clamp" and fl:
        return torch.minimum(torch.maximum(t[1], t[0]), t[2])
    if name == "convert":
        src = args[0].el
        if out_el == "i1":
            return t[0] != 0
        if src in _FLOATS and out_el not in _FLOATS:
            info = torch.iinfo(_tdtype(out_el))
            x = torch.nan_to_num(torch.trunc(t[0].double()), nan=0.0).clamp(info.min, info.max)
            return x.to(_tdtype(out_el))
        return t[0].to(_tdtype(out_el))
    raise _HostOnly(op.name)


def split_experts(arrays, e):
    """Packed arrays whose leading dims multiply to `e` expert slots (a batched
    pack [E, N, ..], or an unbatched one of E * N rows), viewed as [E, N, ..]
    (reference moe.py:1276-1280)."""
    out = []
    for a in arrays:
        rows = count(a.shape[:-1])
        out.append(a.reshape((e, rows // e, a.shape[-1])))
    return out


def pair_indices(indices):
    """(token of pair, expert of pair) for top-k `indices` [T, K]: pair
    p = t * K + j reads token t and expert indices[t, j] (reference
    moe.py:1295-1306, :1432-1433)."""
    import torch
    t, k = indices.shape
    tidx = torch.arange(t, device=indices.device, dtype=torch.int32).repeat_interleave(k)
    return tidx, indices.reshape(t * k).to(torch.int32)


def emit_dot(x, arrays, mode, gs, bits, tidx, eidx, experts, out_dtype=None, has_perm=False):
    """y[p] = x[tidx[p]] . dequant(W[eidx[p]])^T -> [P, (M,) N]
    (reference moe.py:1283-1340, the mx.gather_qmm call at :1320).
    `arrays` are a pack's arrays (w, scales[, biases][, perm]); `x` is [T, K]
    or [T, M, K] (tidx None: row p of x belongs to pair p).  A pack built over
    a permuted contraction axis carries the permutation last: the activations
    are gathered through it first (reference moe.py:1316-1317)."""
    from . import kernels
    biases = arrays[2] if mode == "affine" else None
    if has_perm:
        x = kernels.take_k(x, arrays[-1])
    w, scales = split_experts([arrays[0], arrays[1]], experts)
    if biases is not None:
        (biases,) = split_experts([biases], experts)
    STATS["gather_qmm"] += 1
    return kernels.gather_qmm(x, w, scales, biases, lhs_indices=tidx, rhs_indices=eidx,
                              group_size=gs, bits=bits, mode=mode, out_dtype=out_dtype)


def combine(y_pairs, weights):
    """Routing-weighted sum over each token's K experts, on the device:
    y_pairs [T*K, ...], weights [T, K] -> [T, ...] (reference moe.py:1444-1461)."""
    t, k = weights.shape
    rest = tuple(y_pairs.shape[1:])
    y = y_pairs.reshape((t, k) + rest).float() * weights.reshape((t, k) + (1,) * len(rest)).float()
    return y.sum(dim=1)


def expert_dispatch(interp, match, x, indices, weights):
    """The whole gathered layer for one quantized-matmul match whose weight
    carries the experts: pack lookup, expert-indexed product, weighted sum."""
    from . import qmm
    arrays = qmm.pack_arrays(interp, match)
    experts = count(match.bshape) if match.bshape else match.nshape[0]
    tidx, eidx = pair_indices(indices)
    y = emit_dot(x, arrays, match.mode, match.gs, match.bits, tidx, eidx, experts,
                 out_dtype=qmm._torch_dtype(match.out_dtype), has_perm=match.has_perm)
    STATS["dispatches"] += 1
    return combine(y, weights).to(y.dtype)


# -------------------------------------------------------------- structure ----

def _producer(v):
    return None if v.is_block_arg else v.op


def trace_axes(v, stop_shape=None):
    """Follow `v` down through convert / broadcast_in_dim / transpose / reshapes
    that only add or drop unit axes.  Returns (base, where): where[j] is the
    axis of `v` that base axis j ends up on (None for a unit axis that was
    dropped).  `stop_shape`: stop at the first value of that shape (a caller
    that will READ the base at run time must not look past a convert that the
    dense graph applies)."""
    where = list(range(len(dims_of(v))))
    while True:
        if stop_shape is not None and dims_of(v) == list(stop_shape):
            return v, where
        op = _producer(v)
        if op is None:
            return v, where
        if op.name == "stablehlo.convert":
            v = op.operands[0]
        elif op.name == "stablehlo.broadcast_in_dim":
            where = [where[d] for d in ir.i64_list(op, "broadcast_dimensions")]
            v = op.operands[0]
        elif op.name == "stablehlo.transpose":
            perm = ir.i64_list(op, "permutation")       # result axis i is source axis perm[i]
            src_where = [None] * len(perm)
            for i, p in enumerate(perm):
                src_where[p] = where[i]
            where, v = src_where, op.operands[0]
        elif op.name == "stablehlo.reshape":
            src, dst = dims_of(op.operands[0]), dims_of(op.results[0])
            if [d for d in src if d != 1] != [d for d in dst if d != 1]:
                return v, where
            kept = iter(where[i] for i, d in enumerate(dst) if d != 1)
            where = [None if d == 1 else next(kept) for d in src]
            v = op.operands[0]
        else:
            return v, where


def _splat_value(v):
    op = _producer(v)
    if op is None or op.name != "stablehlo.constant":
        return None
    a = np.asarray(ir.dense_to_np(op.attrs["value"], op.results[0].type))
    return a.reshape(-1)[0] if a.size == 1 else None


def sum_axis(op):
    """The one axis a `reduce(add, init = 0)` sums over."""
    if op is None or op.name != "stablehlo.reduce" or len(op.operands) != 2:
        raise Reject("not a single reduce")
    body = op.attrs.get("body")
    if body is None and op.regions:
        inner = [o for o in op.regions[0].ops if o.name != "return"]
        body = inner[0].name if len(inner) == 1 else None
    if body != "stablehlo.add":
        raise Reject("the reduce does not add")
    axes = list(op.attrs["dimensions"])
    if len(axes) != 1:
        raise Reject("the sum runs over several axes")
    start = _splat_value(op.operands[1])
    if start is None or float(start) != 0.0:
        raise Reject("the sum does not start at zero")
    return axes[0]


def is_top_k(op) -> bool:
    return op is not None and (op.name == "chlo.top_k" or (
        op.name == "stablehlo.composite" and op.attrs.get("name") == "chlo.top_k"))


def top_k_width(op) -> int:
    if op.name == "chlo.top_k":
        return int(op.attrs.get("k", dims_of(op.results[0])[-1]))
    return int(op.attrs.get("composite_attributes", {}).get("k", dims_of(op.results[0])[-1]))


class Router:
    """S [tokens, experts] proven to be `weights` [T, K] scattered at `indices`
    [T, K], which are the index result of `top_k` over logits [T, E]."""
    __slots__ = ("score", "expert_axis", "token_axis", "T", "K", "E", "indices", "weights", "top_k")


def prove_router(score, expert_axis, token_axis) -> Router:
    """`score` (a rank-2 value whose axes `expert_axis` / `token_axis` carry the
    experts and tokens) must be sum_k(one_hot(indices) * weights), built the
    only way a top-k router builds it (reference moe.py:335-442)."""
    r = Router()
    r.score, r.expert_axis, r.token_axis = score, expert_axis, token_axis
    shape = dims_of(score)
    r.E, r.T = shape[expert_axis], shape[token_axis]
    red = _producer(score)
    k_axis = sum_axis(red)
    mul = _producer(red.operands[0])
    while mul is not None and mul.name == "stablehlo.convert":      # a half-precision router sums in float32
        mul = _producer(mul.operands[0])
    if mul is None or mul.name != "stablehlo.multiply":
        raise Reject("the routing scores do not sum a product")
    grid = dims_of(mul.results[0])
    if len(grid) != 3:
        raise Reject("the one-hot product is not rank 3")
    left = [a for a in range(3) if a != k_axis]                     # the reduce keeps these, in order
    e_ax, t_ax = left[expert_axis], left[token_axis]
    r.K = grid[k_axis]
    if (grid[e_ax], grid[t_ax]) != (r.E, r.T):
        raise Reject("the one-hot product and the scores disagree on extents")
    pairs = [r.T, r.K]
    hot_side = None
    for side in (0, 1):
        base, where = trace_axes(mul.operands[side], stop_shape=pairs)
        if where == [t_ax, k_axis] and dims_of(base) == pairs:
            r.weights, hot_side = base, 1 - side
            break
    if hot_side is None:
        raise Reject("no factor of the one-hot product is a [tokens, k] weight")
    cmp_op = _producer(mul.operands[hot_side])
    while cmp_op is not None and cmp_op.name == "stablehlo.convert":
        cmp_op = _producer(cmp_op.operands[0])
    if cmp_op is None or cmp_op.name != "stablehlo.compare" or cmp_op.attrs.get("comparison_direction") != "EQ":
        raise Reject("the one-hot is not an equality comparison")
    if dims_of(cmp_op.results[0]) != grid:
        raise Reject("the one-hot does not have the product's shape")
    index_side = None
    for side in (0, 1):
        base, where = trace_axes(cmp_op.operands[side])
        op = _producer(base)
        if op is not None and op.name == "stablehlo.iota":
            axis = op.attrs["iota_dimension"]
            ishape = dims_of(base)
            if where[axis] == e_ax and ishape[axis] == r.E:
                index_side = 1 - side
                break
    if index_side is None:
        raise Reject("the one-hot compares against no iota over the experts")
    base, where = trace_axes(cmp_op.operands[index_side], stop_shape=pairs)
    if where != [t_ax, k_axis] or dims_of(base) != pairs:
        raise Reject("the one-hot's indices are not laid out [tokens, k]")
    r.indices = base
    # the indices must be a top-k's: another source (a capacity-factor
    # dispatch, say) is a pattern this recognizer has not established
    source, _ = trace_axes(base)
    tk = _producer(source)
    if not is_top_k(tk):
        raise Reject("the routing indices do not come from a top-k")
    if top_k_width(tk) != r.K or dims_of(tk.operands[0]) != [r.T, r.E]:
        raise Reject("the top-k does not select k of [tokens, experts]")
    r.top_k = tk
    return r


# --------------------------------------------------------------- planning ----

def _rest(shape, e, t):
    return [d for i, d in enumerate(shape) if i != e and i != t]


def _rest_pos(e, t, axis):
    """Position of dense axis `axis` among the axes that are neither e nor t."""
    return sum(1 for i in range(axis) if i != e and i != t)


class PairPlan:
    """The region Y of a dispatch re-planned over the selected pairs.

    `lower(value, e, t)` returns the slot that will hold `value` in pair space
    (`[P] + rest`, or its dense self when it has neither axis) and appends the
    closure that fills it.  Closures take a run context with `env` (the
    program's values), `eidx_dev` / `tidx_dev` (expert / token of every pair,
    int64 on the device; `eidx32` / `tidx32` as the kernels take them) and
    `slots` (DevArrays: every closure runs on the device)."""

    def __init__(self, interp, qst, E, T):
        self.interp, self.qst, self.E, self.T = interp, qst, E, T
        self.program = []               # closures, in dependency order
        self.slot_of = {}               # (value, e, t) -> slot
        self.paired = []                # slot -> has a leading pair axis
        self.region = {}                # key -> op: dense ops the dispatch replaces
        self.reads = []                 # values read from env at run time
        self.matches = []               # quantized-matmul matches whose packs are read
        self.dots = 0

    def _new_slot(self, fill, paired) -> int:
        self.program.append(fill)
        self.paired.append(paired)
        return len(self.program) - 1

    def lower(self, v, e, t) -> int:
        at = (v, e, t)
        if at in self.slot_of:
            return self.slot_of[at]
        shape = dims_of(v)
        if e is not None and shape[e] != self.E:
            raise Reject("an expert axis of the wrong extent")
        if t is not None and shape[t] != self.T:
            raise Reject("a token axis of the wrong extent")
        op = _producer(v)
        # THE BOUNDARY: only values that carry the expert axis are region work
        if op is None or e is None:
            slot = self._external(v, e, t)
        elif op.name in ("stablehlo.constant", "stablehlo.iota"):
            raise Reject(f"a per-expert {op.name} inside the region")
        else:
            rule = self._rules.get(op.name) or (PairPlan._elementwise if op.name in _ELEMENTWISE else None)
            if rule is None:
                raise Reject(f"{op.name} is not modelled over pairs")
            self.region[op_key(op)] = op
            slot = rule(self, op, e, t)
        self.slot_of[at] = slot
        return slot

    # -- values from outside the region: gathered on the way in
    def _external(self, v, e, t):
        op = _producer(v)
        fixed = []                        # a constant is evaluated when planned and uploaded once
        if op is not None and op.name == "stablehlo.constant":
            out = REGISTRY[op.name](self.interp, op, [], {})
            fixed.append(out[0] if isinstance(out, (list, tuple)) else out)
        else:
            self.reads.append(v)

        def fill(ctx):
            if fixed:
                if not isinstance(fixed[0], DevArray):
                    fixed[0] = dev(fixed[0])
                a = fixed[0]
            else:
                a = dev(ctx.env[v])
            if e is None and t is None:
                return a
            x = a.t
            if e is not None and t is not None:
                x = x.movedim((e, t), (0, 1))[ctx.eidx_dev, ctx.tidx_dev]
            elif e is not None:
                x = x.movedim(e, 0).index_select(0, ctx.eidx_dev)
            else:
                x = x.movedim(t, 0).index_select(0, ctx.tidx_dev)
            return DevArray(x, a.el)
        return self._new_slot(fill, e is not None or t is not None)

    def _lead(self, slot, a, P):
        """A slot's tensor with a leading pair axis of extent P or 1."""
        return a if self.paired[slot] else a.reshape((1,) + tuple(a.shape))

    # -- shape-preserving ops
    def _elementwise(self, op, e, t):
        shape = dims_of(op.results[0])
        ins = []
        for x in op.operands:
            xs = dims_of(x)
            if xs == shape:
                ins.append(self.lower(x, e, t))
            elif not xs:
                ins.append(self.lower(x, None, None))
            else:
                raise Reject(f"{op.name} mixes shapes {xs} and {shape}")
        handler = REGISTRY[op.name]
        out_el = elem(op.results[0])

        def fill(ctx):
            args = []
            for s in ins:
                h = ctx.slots[s]
                # an unpaired full-shape operand (a splat) broadcasts along the pair axis
                if not self.paired[s] and h.t.dim():
                    h = DevArray(h.t.reshape((1,) + tuple(h.t.shape)), h.el)
                args.append(h)
            try:
                return DevArray(_dev_elementwise(op, args, out_el), out_el)
            except _HostOnly:
                out = handler(self.interp, op, [host(a.t) for a in args], {})
                return dev(out[0] if isinstance(out, (list, tuple)) else out)
        return self._new_slot(fill, True)

    def _concatenate(self, op, e, t):
        axis = op.attrs.get("dim", op.attrs.get("dimension"))
        if axis in (e, t):
            raise Reject("a concatenation along the expert or token axis")
        ins = [self.lower(x, e, t) for x in op.operands]
        pos = 1 + _rest_pos(e, t, axis)

        def fill(ctx):
            import torch
            parts = [self._lead(s, ctx.slots[s].t, ctx.P) for s in ins]
            lead = max(p.shape[0] for p in parts)
            parts = [p.expand((lead,) + tuple(p.shape[1:])) for p in parts]
            return DevArray(torch.cat(parts, dim=pos), ctx.slots[ins[0]].el)
        return self._new_slot(fill, True)

    # -- shape ops
    def _broadcast(self, op, e, t):
        placement = ir.i64_list(op, "broadcast_dimensions")
        if placement != sorted(placement):
            raise Reject("a broadcast that also permutes")
        src = op.operands[0]
        sshape, shape = dims_of(src), dims_of(op.results[0])
        se = st = None
        dropped = set()
        for j, d in enumerate(placement):
            if d not in (e, t):
                continue
            full = self.E if d == e else self.T
            # a unit source axis is a broadcast, never the axis itself (the two
            # readings coincide when T = 1, every decode step, and reading it as
            # the token axis would demand one of everything upstream)
            if sshape[j] == 1:
                dropped.add(j)
            elif sshape[j] == full:
                if d == e:
                    se = j
                else:
                    st = j
            else:
                raise Reject("the expert / token axis is broadcast from a part of it")
        inner = self.lower(src, se, st)
        out_rest = _rest(shape, e, t)
        spots = []                       # for each kept source axis: its position in out_rest
        for j in range(len(sshape)):
            if j in (se, st):
                continue
            spots.append(None if j in dropped else _rest_pos(e, t, placement[j]))

        def fill(ctx):
            h = ctx.slots[inner]
            a = self._lead(inner, h.t, ctx.P)
            index = [slice(None)] + [0 if s is None else slice(None) for s in spots]
            a = a[tuple(index)]
            view = [1] * len(out_rest)
            for s, extent in zip([s for s in spots if s is not None], a.shape[1:]):
                view[s] = extent
            a = a.reshape([a.shape[0]] + view)
            return DevArray(a.expand([a.shape[0]] + out_rest), h.el)
        return self._new_slot(fill, True)

    def _transpose(self, op, e, t):
        perm = ir.i64_list(op, "permutation")
        src = op.operands[0]
        se = perm[e] if e is not None else None
        st = perm[t] if t is not None else None
        inner = self.lower(src, se, st)
        order = [_rest_pos(se, st, perm[i]) for i in range(len(perm)) if i not in (e, t)]

        def fill(ctx):
            h = ctx.slots[inner]
            a = self._lead(inner, h.t, ctx.P)
            return DevArray(a.permute([0] + [1 + i for i in order]), h.el)
        return self._new_slot(fill, True)

    def _reshape(self, op, e, t):
        src = op.operands[0]
        sshape, shape = dims_of(src), dims_of(op.results[0])
        head = max(a for a in (e, t) if a is not None) + 1
        if len(sshape) < head or sshape[:head] != shape[:head]:
            raise Reject("a reshape across the expert / token axes")
        inner = self.lower(src, e, t)
        out_rest = _rest(shape, e, t)

        def fill(ctx):
            h = ctx.slots[inner]
            a = self._lead(inner, h.t, ctx.P)
            return DevArray(a.reshape([a.shape[0]] + out_rest), h.el)
        return self._new_slot(fill, True)

    def _slice(self, op, e, t):
        src = op.operands[0]
        sshape = dims_of(src)
        b, l, s = op.attrs["start_indices"], op.attrs["limit_indices"], op.attrs["strides"]
        for a in (e, t):
            if a is not None and (b[a], l[a], s[a]) != (0, sshape[a], 1):
                raise Reject("a slice cuts the expert or token axis")
        inner = self.lower(src, e, t)
        cut = tuple(slice(b[i], l[i], s[i]) for i in range(len(sshape)) if i not in (e, t))

        def fill(ctx):
            h = ctx.slots[inner]
            a = self._lead(inner, h.t, ctx.P)
            return DevArray(a[(slice(None),) + cut], h.el)
        return self._new_slot(fill, True)

    # -- the per-expert products
    def _packed(self, dot, weight_side):
        """The quantized-matmul match that fused this dot."""
        for m in self.qst.matches:
            if m.key is not op_key(dot) or m.disabled:
                continue
            if m.swapped != (weight_side == 0):
                raise Reject("the quantized operand of the dot is not the per-expert weight")
            if len(m.bshape) > 1 or (m.bshape and m.bshape[0] != self.E):
                raise Reject("the pack's batch axis is not the expert axis")
            if not m.bshape and (not m.nshape or m.nshape[0] != self.E):
                raise Reject("the experts are not the leading axis of the packed rows")
            return m
        raise Reject("a per-expert dot whose weight is not a packed quantized weight")

    def _dot(self, op, e, t):
        lb, rb, lc, rc = ir.dot_dims(op)
        lhs, rhs = op.operands
        lshape, rshape = dims_of(lhs), dims_of(rhs)
        lfree = [d for d in range(len(lshape)) if d not in lb and d not in lc]
        rfree = [d for d in range(len(rshape)) if d not in rb and d not in rc]
        nb = len(lb)
        if t is None:
            raise Reject("a per-expert dot without a token axis")

        def origin(axis):
            """(side, operand axis) of a result axis; side 2: a batch axis of both."""
            if axis < nb:
                return 2, axis
            if axis < nb + len(lfree):
                return 0, lfree[axis - nb]
            return 1, rfree[axis - nb - len(lfree)]

        e_side, e_dim = origin(e)
        t_side, t_dim = origin(t)
        if t_side == 2:
            raise Reject("the token axis is a batch axis of the dot")
        data_side, weight_side = t_side, 1 - t_side
        if e_side == 2:
            data_e = (lb, rb)[data_side][e_dim]
        elif e_side == weight_side:
            data_e = None
        else:
            raise Reject("only the activations carry the expert axis")
        m = self._packed(op, weight_side)
        data = op.operands[data_side]
        dshape = dims_of(data)
        dbatch, dcontract = (lb, rb)[data_side], (lc, rc)[data_side]
        dfree = [d for d in range(len(dshape)) if d not in dbatch and d not in dcontract]
        row_axes = [d for d in dfree if d != t_dim]                  # activation rows of one pair
        M = count(dshape[d] for d in row_axes)
        if M != m.M // self.T:
            raise Reject("the match and the dispatch disagree on the rows of a pair")
        wfree = (lfree, rfree)[weight_side]
        n_axes = [d for d in wfree if not (e_side == weight_side and d == e_dim)]
        nshape = [dims_of(op.operands[weight_side])[d] for d in n_axes]
        N, K = count(nshape), m.K
        mshape = [dshape[d] for d in row_axes]
        # gather_qmm returns [P] + rows + columns; the dense result lists batch,
        # lhs-free, rhs-free axes
        shape = dims_of(op.results[0])
        order = []
        for i in range(len(shape)):
            if i in (e, t):
                continue
            side, dim = origin(i)
            if side == 2:
                raise Reject("a batch axis besides the experts in a per-expert dot")
            order.append(row_axes.index(dim) if side == data_side else len(row_axes) + n_axes.index(dim))
        out_rest = _rest(shape, e, t)
        # activations: token-indexed and nothing else -> hand the kernel the
        # ungathered rows and the pairs' token numbers (no K-fold copy)
        data_op = _producer(data)
        direct = data_e is None and (data_op is None or op_key(data_op) not in self.region)
        if direct:
            self.reads.append(data)
            inner = None
        else:
            inner = self.lower(data, data_e, t_dim)
        # data in pair space is [P] + (data axes without e, t) = rows.. and contraction axes in dense order
        data_rest_axes = [d for d in range(len(dshape)) if d not in (data_e, t_dim)]
        to_rows_k = [data_rest_axes.index(d) for d in row_axes + list(dcontract)]
        self.matches.append(m)
        self.dots += 1
        out_el = elem(op.results[0])
        E, T = self.E, self.T

        def fill(ctx):
            from . import qmm
            import torch
            if direct:
                dense = qmm.to_device(ctx.env[data])
                dense = dense.permute([t_dim] + [d for d in row_axes + list(dcontract)])
                x = dense.reshape(T, M, K)
                lhs = ctx.tidx32
            else:
                h = ctx.slots[inner]                 # the previous slot as it lies on the device
                a = self._lead(inner, h.t, ctx.P)
                a = a.expand((ctx.P,) + tuple(a.shape[1:]))
                x = a.permute([0] + [1 + i for i in to_rows_k]).reshape(ctx.P, M, K)
                lhs = None
            if x.dtype not in (torch.float32, torch.float16, torch.bfloat16):
                x = x.to(qmm._torch_dtype(out_el))
            arrays = qmm.pack_arrays(ctx.interp, m)
            y = emit_dot(x.contiguous(), arrays, m.mode, m.gs, m.bits, lhs, ctx.eidx32, E,
                         out_dtype=qmm._torch_dtype(out_el), has_perm=m.has_perm)
            y = y.reshape([ctx.P] + mshape + nshape)
            if order != sorted(order):
                y = y.permute([0] + [1 + i for i in order])
            return DevArray(y.reshape([ctx.P] + out_rest), out_el)
        return self._new_slot(fill, True)

    _rules = {"stablehlo.concatenate": _concatenate, "stablehlo.broadcast_in_dim": _broadcast,
              "stablehlo.transpose": _transpose, "stablehlo.reshape": _reshape,
              "stablehlo.slice": _slice, "stablehlo.dot_general": _dot}


class _Run:
    __slots__ = ("interp", "env", "slots", "P", "eidx_dev", "tidx_dev", "eidx32", "tidx32")


class Dispatch:
    """One gathered expert dispatch: replaces `root` (named by `key`), skips
    `skip_keys`, reads `reads` (+ the router's indices and weights) from env."""

    def __init__(self):
        self.disabled = False
        self.verified = not VERIFY
        self._tidx = None

    def run(self, interp, env):
        """The closure list on the device, then the routing-weighted sum over
        each token's K pairs.  The only host data read are the router's indices
        when the program computed them on the host (an upload, no copy back)."""
        import torch
        from . import qmm
        from .interpreter import HOST_COPIES
        copies = HOST_COPIES[0]
        r, plan = self.router, self.plan
        ctx = _Run()
        ctx.interp, ctx.env, ctx.P = interp, env, self.P
        iv = env[r.indices]
        if hasattr(iv, "type_enum") and hasattr(iv, "data"):
            iv = iv.data
        if isinstance(iv, torch.Tensor):
            ctx.eidx32 = qmm.to_device(iv).reshape(-1).to(torch.int32)
        else:
            ctx.eidx32 = torch.from_numpy(np.ascontiguousarray(host(iv).a.reshape(-1), np.int32)).to(qmm.DEVICE)
        if self._tidx is None:                      # token of pair p: p // K, the same every call
            t32 = torch.arange(self.T, dtype=torch.int32, device=qmm.DEVICE).repeat_interleave(self.K)
            self._tidx = (t32, t32.long())
        ctx.tidx32, ctx.tidx_dev = self._tidx
        ctx.eidx_dev = ctx.eidx32.long()
        ctx.slots = []
        for fill in plan.program:
            ctx.slots.append(fill(ctx))
        out = ctx.slots[self.out_slot]
        yd = out.t
        if not plan.paired[self.out_slot]:
            yd = yd.reshape((1,) + tuple(yd.shape))
        yd = yd.expand((self.P,) + tuple(yd.shape[1:]))
        wd = qmm.to_device(env[r.weights]).reshape(self.T, self.K)
        if self.sum_el != out.el:
            yd = yd.to(qmm._torch_dtype(self.sum_el))         # the dense graph converts the products before summing
        total = combine(yd, wd)
        if self.out_axis:
            total = torch.movedim(total, 0, self.out_axis)
        if list(total.shape) != self.out_shape:
            raise RuntimeError(f"expert dispatch produced {list(total.shape)}, expected {self.out_shape}")
        STATS["dispatches"] += 1
        STATS["host_copies"] += HOST_COPIES[0] - copies
        return [total.to(qmm._torch_dtype(self.out_el))]


Match = Dispatch            # the reference's name for a gathered dispatch (moe.py; qmm.py:670)


def plan_root(interp, qst, block, root) -> Dispatch:
    """`root` as the weighted sum over the experts of a dense dispatch."""
    e_axis = sum_axis(root)
    mul, casts = _producer(root.operands[0]), []
    while mul is not None and mul.name == "stablehlo.convert":       # a half-precision model sums in float32
        casts.append(mul)
        mul = _producer(mul.operands[0])
    if mul is None or mul.name != "stablehlo.multiply":
        raise Reject("the sum over experts does not add up a product")
    grid = dims_of(mul.results[0])
    if len(grid) < 2:
        raise Reject("the expert product has fewer than two axes")
    router = t_axis = y = None
    for side in (0, 1):
        base, where = trace_axes(mul.operands[side])
        if len(where) != 2 or e_axis not in where:
            continue
        se = where.index(e_axis)
        st = 1 - se
        if where[st] is None or where[st] == e_axis:
            continue
        router = prove_router(base, se, st)
        t_axis, y = where[st], mul.operands[1 - side]
        break
    if router is None:
        raise Reject("no factor of the expert product is a routing-score tensor")
    if (grid[e_axis], grid[t_axis]) != (router.E, router.T):
        raise Reject("the routing scores and the expert outputs disagree on extents")
    g = Dispatch()
    g.root, g.key, g.router = root, op_key(root), router
    g.E, g.T, g.K, g.P = router.E, router.T, router.K, router.T * router.K
    g.out_shape = [d for i, d in enumerate(grid) if i != e_axis]
    g.out_axis = sum(1 for i in range(t_axis) if i != e_axis)         # where the token axis sits in the result
    g.out_el, g.sum_el = elem(root.results[0]), elem(root.operands[0])
    plan = PairPlan(interp, qst, router.E, router.T)
    plan.region[op_key(mul)] = mul
    for c in casts:
        plan.region[op_key(c)] = c
    g.out_slot = plan.lower(y, e_axis, t_axis)
    if not plan.dots:
        raise Reject("no per-expert dot in the region")
    # a region op may only vanish if nothing outside the region reads it
    for key, op in plan.region.items():
        for res in op.results:
            for user in res.uses:
                ukey = op_key(user)
                if ukey is not g.key and (ukey is None or ukey not in plan.region):
                    raise Reject(f"{op.name} is also read outside the region ({user.name})")
    for v in plan.reads:
        op = _producer(v)
        if op is not None and op_key(op) in plan.region:
            raise Reject(f"{op.name} is both region work and a run-time read")
    g.plan, g.reads = plan, list(plan.reads)
    g.matches = list(dict.fromkeys(plan.matches))
    g.skip_keys = frozenset(sweep_dead(block, set(plan.region), g))
    g.name = f"E{g.E}/K{g.K}/T{g.T}->" + "x".join(str(d) for d in g.out_shape)
    g.bytes = sum(count(dims_of(op.results[0])) * ir._EL_BYTES[elem(op.results[0])] * g.P // max(1, g.E * g.T)
                  for op in plan.region.values() if op.results)
    return g


def sweep_dead(block, skip, g):
    """Besides the region itself, the dense ops that only the replaced sum
    ever read (the [tokens, experts] scores, the one-hot, their broadcasts)
    need not run.  Definitions precede uses in a block, so one walk from the
    last op to the first sees every reader of an op before the op."""
    keep = set()                          # what the dispatch still reads, and everything that computes it
    todo = list(g.reads) + [g.router.indices, g.router.weights]
    while todo:
        v = todo.pop()
        if v in keep:
            continue
        keep.add(v)
        op = _producer(v)
        if op is not None:
            todo.extend(op.operands)
    for op in reversed(block.ops):
        key = op_key(op)
        if key is None or key in skip or key is g.key or op.name in OPAQUE_OPS or op.regions and op.name != "stablehlo.reduce":
            continue
        if any(res in keep for res in op.results):
            continue
        readers = [user for res in op.results for user in res.uses]
        if readers and all(op_key(u) is g.key or op_key(u) in skip for u in readers):
            skip.add(key)
    return skip


def plan_dispatches(interp, qst):
    """Every gatherable dispatch of the program (reference moe.py:1022-1090);
    the quantized-matmul matches they read are marked absorbed."""
    if not ENABLED:
        return []
    found = []
    for block in ir.walk_blocks(interp._main_block()):
        for op in block.ops:
            if op.name != "stablehlo.reduce":
                continue
            try:
                found.append(plan_root(interp, qst, block, op))
            except Reject as why:
                if len(dims_of(op.operands[0])) >= 3:
                    _debug(f"a sum over {dims_of(op.operands[0])} is not a gatherable dispatch ({why})")
    kept, taken = [], set()
    for g in found:
        if g.key in taken or g.skip_keys & taken:
            continue
        taken |= set(g.skip_keys) | {g.key}
        kept.append(g)
    for g in kept:
        for m in g.matches:
            m.absorbed = True
    STATS["recognized"] += len(kept)
    if kept:
        _debug(f"{len(kept)} expert dispatch(es) gathered ({', '.join(g.name for g in kept)})")
    return kept


def analyze(interp, qst):
    """The reference's entry point under its own name (moe.py:1016-1090): find
    the gatherable dispatches and extend the recognizer's state with them."""
    qst.moe = plan_dispatches(interp, qst)


# ----------------------------------------------------------- verification ----

def verify(interp, g):
    """S == scatter(w at idx) on random logits, a few draws (the later ones on
    coarse values: exact ties are where a top-k and a hand-rolled scatter
    would most easily disagree).  The router tail below the top-k depends on
    nothing but the logits, so this checks the structural reading -- which
    axis is which, and that the weights land at the matched indices -- without
    any real activation (reference moe.py:1112-1153)."""
    from .packs import evaluate
    r = g.router
    logits = r.top_k.operands[0]
    rng = np.random.default_rng(20260803)
    rows = np.repeat(np.arange(g.T), g.K)
    for draw in range(max(1, VERIFY_DRAWS)):
        raw = rng.standard_normal((g.T, g.E)).astype(np.float32)
        if draw:
            raw = np.round(raw * 2.0) / 2.0
        env = {logits: settle(raw, elem(logits))}
        score = host(evaluate(interp, r.score, env)).a.astype(np.float64)
        idx = host(evaluate(interp, r.indices, env)).a.reshape(-1).astype(np.int64)
        wgt = host(evaluate(interp, r.weights, env)).a.reshape(-1).astype(np.float64)
        if r.expert_axis == 0:
            score = score.T
        if list(score.shape) != [g.T, g.E]:
            raise Reject(f"the routing scores evaluate to shape {list(score.shape)}")
        want = np.zeros((g.T, g.E))
        np.add.at(want, (rows, idx), wgt)
        if not np.array_equal(score, want):
            raise Reject("the routing scores are not the top-k weights scattered at the matched indices")
        if int((score != 0).sum(axis=1).max()) > g.K:
            raise Reject(f"a token has more than {g.K} nonzero routing weights")
    STATS["verified"] += 1


def prologue(interp, st) -> bool:
    """Disable dispatches whose expert weight did not pack, verify the rest
    once.  True when the rewrite changed (reference moe.py:1156-1190)."""
    changed = False
    for g in st.moe:
        if g.disabled:
            continue
        why = None
        if any(m.disabled for m in g.matches):
            why = "its quantized weight did not pack"
        elif not g.verified:
            try:
                verify(interp, g)
                g.verified = True
            except Exception as e:
                why = str(e)
        if why is not None:
            g.disabled = changed = True
            STATS["fallbacks"] += 1
            _debug(f"{g.name} falls back to the dense dispatch ({why})")
            for m in g.matches:
                m.absorbed = False
    return changed


# ---- hooks the interpreter reaches through qmm's root dispatch

def emit_reads(g):
    """Everything `emit` reads out of env: what the plan gathers on the way
    into the region, and the router's two tensors."""
    return tuple(g.reads) + (g.router.indices, g.router.weights)


def emit_bytes(g) -> int:
    return int(getattr(g, "bytes", 0))


def emit(interp, g, env):
    return g.run(interp, env)
