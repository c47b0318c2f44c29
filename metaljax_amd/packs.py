"""Value half of the quantized-matmul recognizer: evaluate a match's operand
subtrees on concrete buffers, verify that the weight really is what the fused
kernel will compute, and pack it.

Same job and outcomes as the reference's pack step (reference
src/metaljax/qmm.py:1130-2302: `_eval`, `_Source`, `_build_*_pack`, the build
cache, `_share`, `_resolve`); the formulation is this package's own.

  * `WeightRows` hands the builders an operand as `[rows, K]` matrices, either
    whole or one block of the weight's leading axis at a time.  For the
    blocked form the subtree is compiled once into a `_Tape` -- a straight list
    of steps, each marked as "per block" (it keeps the blocked axis and is
    row-local) or "once" (block-independent: a decode table, a splat) -- and
    the tape is replayed per block.  Anything that is not provably row-local
    raises `NotBlockable` and the weight is evaluated whole instead; both ways
    give bit-identical packs (reference tests/test_qmm.py:964-988, :1029-1057).
  * The builders are made of passes over the blocks (`_CodeRange`,
    `_GroupTables`, then the packing pass): what has to be decided for the
    whole weight (code width and offset, group size) is reduced over the
    blocks first, so no block's decision depends on which block it is.
  * Packs are remembered three ways: per match by the identity of the buffers
    they were built from, across executables by (subtree text, buffers), and
    by content (tied or duplicated weights share device arrays).

Packing runs in numpy on the host; the packed arrays are uploaded once.
"""

from __future__ import annotations

import hashlib
import os
import weakref

import numpy as np

from . import ir, packing
from .interpreter import REGISTRY, HostArray, host
from .packing import BF16Array, Reject
from .recognize import OPAQUE_OPS, count, dims_of, outer_definition

MAX_PACKS = int(os.environ.get("METALJAX_QMM_CACHE", "2"))
MAX_REPACKS = int(os.environ.get("METALJAX_QMM_REPACKS", "8"))
# Entries the two pack tables keep (0 turns the table off; reference qmm.py:1653, :2209-2211).
# Entries are weak, so a full table is first swept of its dead ones and only then dropped whole --
# coarse, and it only ever costs a repack.
MAX_SHARED = int(os.environ.get("METALJAX_QMM_SHARE", "512"))
MAX_BUILT = int(os.environ.get("METALJAX_QMM_BUILD_CACHE", "512"))
# Weight elements evaluated per block (reference qmm.py:1259): the chain that
# rebuilds a weight is several times wider than the weight.
BLOCK_ELEMS = int(os.environ.get("METALJAX_QMM_BLOCK", str(1 << 24)))
# Largest block-independent value a blocked evaluation accepts (a bigger one
# means the blocking misread the graph).
WHOLE_MAX = 1 << 22

STATS = {"recognized": 0, "packs": 0, "fallbacks": 0, "perms": 0, "mxfp4": 0, "batched": 0,
         "shared": 0, "blocked": 0, "build_hits": 0, "build_declines": 0}

_debug = lambda text: None            # replaced by qmm when METALJAX_DEBUG=1


class NotBlockable(Exception):
    """The subtree cannot be evaluated one row block at a time.  Not a Reject:
    the weight still packs, from a whole evaluation."""


# ------------------------------------------------------ whole evaluation ----

def evaluate(interp, value, env):
    """`value` computed from the values bound in `env` (usually @main's
    arguments) with the interpreter's own handlers; results are added to
    `env`.  Iterative, since reconstruction chains can be long."""
    pending = [value]
    while pending:
        v = pending[-1]
        if v in env:
            pending.pop()
            continue
        if v.is_block_arg:
            outside = outer_definition(v)
            if outside is v:
                raise Reject("a value of the weight's subtree is not bound")
            if outside in env:
                env[v] = env[outside]
                pending.pop()
            else:
                pending.append(outside)
            continue
        op = v.op
        unready = [x for x in op.operands if x not in env]
        if unready:
            pending.extend(unready)
            continue
        run = REGISTRY.get(op.name)
        if run is None or op.name in OPAQUE_OPS:
            raise Reject(f"{op.name} cannot be evaluated at pack time")
        produced = run(interp, op, [env[x] for x in op.operands], env)
        if not isinstance(produced, (list, tuple)):
            produced = [produced]
        for res, val in zip(op.results, produced):
            env[res] = val
        pending.pop()
    return env[value]


def apply_shape_ops(a: np.ndarray, ops):
    for op in ops:
        if op.name == "stablehlo.reshape":
            a = a.reshape(op.results[0].type.shape)
        else:
            a = np.transpose(a, ir.i64_list(op, "permutation"))
    return a


def as_rows(x: HostArray, m) -> np.ndarray:
    """A tensor shaped like the dot's quantized operand (before the match's
    shape ops) as the `[B * N, K]` matrix the kernels' layout is made of."""
    a = apply_shape_ops(x.a, m.post)
    if list(a.shape) != m.rshape:
        raise Reject(f"the operand evaluates to shape {list(a.shape)}, the dot reads {m.rshape}")
    return np.ascontiguousarray(np.transpose(a, m.rperm).reshape(-1, m.K))


# ---------------------------------------------------- blocked evaluation ----

ROWS, ONCE = "rows", "once"

# Ops whose handler computes each result element from the same element of its
# operands and never reads the result type's shape: a block of the operands
# gives that block of the result.
_ELEMENTWISE = frozenset("""
    stablehlo.abs stablehlo.add stablehlo.and stablehlo.ceil stablehlo.clamp stablehlo.compare
    stablehlo.convert stablehlo.divide stablehlo.exponential stablehlo.floor stablehlo.log
    stablehlo.logistic stablehlo.maximum stablehlo.minimum stablehlo.multiply stablehlo.negate
    stablehlo.not stablehlo.or stablehlo.power stablehlo.round_nearest_even stablehlo.rsqrt
    stablehlo.select stablehlo.shift_left stablehlo.shift_right_arithmetic
    stablehlo.shift_right_logical stablehlo.sign stablehlo.sqrt stablehlo.subtract stablehlo.tanh
    stablehlo.xor
""".split())
# Ops with no operands to block: evaluated once and cut into rows
_SOURCES = frozenset({"stablehlo.constant", "stablehlo.iota"})


class _Step:
    __slots__ = ("kind", "op", "ins", "when", "arg")

    def __init__(self, kind, when, op=None, ins=(), arg=None):
        self.kind, self.when, self.op, self.ins, self.arg = kind, when, op, tuple(ins), arg


class _Tape:
    """One operand subtree compiled for evaluation by blocks of `lead` rows.

    Compilation walks down from the root with a demand -- ROWS (this block of
    the value's leading axis) or ONCE (all of it, the same for every block) --
    and every op decides from its own attributes what it demands of its
    operands; a value wanted both ways gets two steps.  A call is compiled
    inside its callee (its body's shapes are declared for the full extent), a
    loop carry is followed outwards.  Replaying runs the ONCE steps on first
    use and the ROWS steps for every block."""

    def __init__(self, interp, args, arg_number, lead, root):
        self.interp, self.args, self.arg_number, self.lead = interp, args, arg_number, lead
        self.steps = []                  # in execution order
        self.where = {}                  # (frame, value, demand) -> (step number, result number)
        self.frames = {0: (None, {})}    # frame -> (calling frame, {callee argument: call operand})
        self.depth = 0
        self.root = self._want(root, ROWS, 0)
        self.once_values = {}

    # -- compilation
    def _emit(self, step) -> int:
        self.steps.append(step)
        return len(self.steps) - 1

    def _want(self, value, demand, frame):
        at = (frame, value, demand)
        got = self.where.get(at)
        if got is not None:
            return got
        self.depth += 1
        if self.depth > 400:
            raise NotBlockable("the subtree is too deep to compile")
        try:
            got = self._compile(value, demand, frame)
        finally:
            self.depth -= 1
        self.where[at] = got
        return got

    def _compile(self, value, demand, frame):
        if value.is_block_arg:
            caller, bound = self.frames[frame]
            if value in bound:
                return self._want(bound[value], demand, caller)
            number = self.arg_number.get(value)
            if number is None:
                outside = outer_definition(value)
                if outside is value:
                    raise Reject("a value of the weight's subtree is not bound")
                return self._want(outside, demand, frame)
            if demand == ROWS:
                shape = dims_of(value)
                if not shape or shape[0] != self.lead:
                    raise NotBlockable(f"argument {number} does not have the blocked axis")
            return self._emit(_Step("arg", demand, arg=number)), 0
        op = value.op
        if op.name in OPAQUE_OPS or op.name not in REGISTRY:
            raise Reject(f"{op.name} cannot be evaluated at pack time")
        if demand == ONCE:
            if any(dims_of(r) and count(dims_of(r)) > WHOLE_MAX for r in op.results):
                raise NotBlockable(f"{op.name} is the same for every block but has more than {WHOLE_MAX} elements")
            ins = [self._want(x, ONCE, frame) for x in op.operands]
            return self._emit(_Step("op", ONCE, op, ins)), value.index
        # demand == ROWS
        out_shape = dims_of(value)
        if not out_shape or out_shape[0] != self.lead:
            raise NotBlockable(f"{op.name} does not keep the blocked axis")
        if op.name == "func.call":
            callee = self.interp.module.funcs.get(op.attrs.get("callee"))
            if callee is None:
                raise NotBlockable("call of an unknown function")
            body = callee.body
            inner = len(self.frames)
            self.frames[inner] = (frame, dict(zip(body.args, op.operands)))
            return self._want(body.terminator.operands[value.index], ROWS, inner)
        return self._emit(self._row_step(op, frame)), value.index

    def _carries_rows(self, v) -> bool:
        shape = dims_of(v)
        return bool(shape) and shape[0] == self.lead

    def _row_step(self, op, frame) -> _Step:
        name, lead = op.name, self.lead
        want = lambda v, demand: self._want(v, demand, frame)
        if name in _SOURCES:
            whole = self._want(op.results[0], ONCE, frame)
            return _Step("cut", ROWS, op, [whole])
        if name == "stablehlo.reshape":
            src, out = dims_of(op.operands[0]), dims_of(op.results[0])
            if not src or src[0] != lead or count(src[1:]) != count(out[1:]):
                raise NotBlockable("a reshape folds the blocked axis into others")
            return _Step("reshape", ROWS, op, [want(op.operands[0], ROWS)])
        if name == "stablehlo.broadcast_in_dim":
            src = dims_of(op.operands[0])
            placement = ir.i64_list(op, "broadcast_dimensions")
            # the operand is blocked only if its own leading axis becomes the
            # result's; a leading extent of 1 stretched to `lead` is one row
            # that every block reads whole
            blocked = bool(placement) and placement[0] == 0 and bool(src) and src[0] == lead
            if not blocked and 0 in placement and src[placement.index(0)] not in (1,):
                raise NotBlockable("a broadcast puts another axis on the blocked one")
            return _Step("broadcast", ROWS, op, [want(op.operands[0], ROWS if blocked else ONCE)],
                         arg=blocked)
        if name == "stablehlo.slice":
            if (op.attrs["start_indices"][0] != 0 or op.attrs["limit_indices"][0] != lead
                    or op.attrs["strides"][0] != 1):
                raise NotBlockable("a slice cuts the blocked axis")
            return _Step("slice", ROWS, op, [want(op.operands[0], ROWS)])
        if name == "stablehlo.transpose":
            if ir.i64_list(op, "permutation")[0] != 0:
                raise NotBlockable("a transpose moves the blocked axis")
            return _Step("op", ROWS, op, [want(op.operands[0], ROWS)])
        if name == "stablehlo.concatenate":
            if op.attrs.get("dim", op.attrs.get("dimension")) == 0:
                raise NotBlockable("a concatenation along the blocked axis")
            return _Step("op", ROWS, op, [want(x, ROWS) for x in op.operands])
        if name == "stablehlo.gather":
            # a table lookup (jax's `take`): the indices carry the block, the
            # table is the same for every block
            dn = op.attrs["dimension_numbers"][1]
            idx_shape = dims_of(op.operands[1])
            if (0 in dn.get("offset_dims", []) or dn.get("index_vector_dim", len(idx_shape) - 1) == 0
                    or dn.get("operand_batching_dims") or not idx_shape or idx_shape[0] != lead):
                raise NotBlockable("a gather whose indices do not run along the blocked axis")
            return _Step("gather", ROWS, op, [want(op.operands[0], ONCE), want(op.operands[1], ROWS)])
        if name == "stablehlo.reduce":
            if 0 in tuple(op.attrs["dimensions"]):
                raise NotBlockable("a reduction over the blocked axis")
            half = len(op.operands) // 2
            return _Step("op", ROWS, op, [want(x, ROWS) for x in op.operands[:half]]
                         + [want(x, ONCE) for x in op.operands[half:]])
        if name in _ELEMENTWISE:
            # operands have the result's shape, except rank-0 ones (a select's
            # predicate, a clamp's bounds), which every block reads whole
            return _Step("op", ROWS, op, [want(x, ROWS if self._carries_rows(x) else ONCE)
                                          for x in op.operands])
        raise NotBlockable(f"{name} is not known to be row-local")

    # -- replay
    def block(self, lo, hi) -> np.ndarray:
        rows = hi - lo
        vals = {}

        def value_of(ref):
            number, res = ref
            step = self.steps[number]
            store = self.once_values if step.when == ONCE else vals
            return store[number][res]

        for number, step in enumerate(self.steps):
            store = self.once_values if step.when == ONCE else vals
            if number in store:
                continue
            store[number] = self._run(step, [value_of(r) for r in step.ins], lo, hi, rows)
        out = host(value_of(self.root))
        if out.a.shape[0] != rows:
            raise NotBlockable(f"a block of {rows} rows evaluated to {list(out.a.shape)}")
        return out.a

    def _run(self, step, ins, lo, hi, rows):
        kind, op = step.kind, step.op
        if kind == "arg":
            h = host(self.args[step.arg])
            return [h if step.when == ONCE else HostArray(h.a[lo:hi], h.el)]
        if kind == "cut":
            h = host(ins[0])
            return [HostArray(h.a[lo:hi], h.el)]
        if kind == "reshape":
            h = host(ins[0])
            return [HostArray(h.a.reshape([rows] + dims_of(op.results[0])[1:]), h.el)]
        if kind == "slice":
            h = host(ins[0])
            cut = (slice(None),) + tuple(slice(b, e, s) for b, e, s in zip(
                op.attrs["start_indices"][1:], op.attrs["limit_indices"][1:], op.attrs["strides"][1:]))
            return [HostArray(h.a[cut], h.el)]
        if kind == "broadcast":
            h = host(ins[0])
            out = [rows] + dims_of(op.results[0])[1:]
            spread = [1] * len(out)
            for axis, where in enumerate(ir.i64_list(op, "broadcast_dimensions")):
                spread[where] = h.a.shape[axis]
            if spread[0] not in (1, rows):
                raise NotBlockable("a broadcast stretches the blocked axis")
            return [HostArray(np.broadcast_to(h.a.reshape(spread), out), h.el)]
        if kind == "gather":
            # the handler shapes its result by the declared type: give it that
            # type's rows only
            produced = _gather_rows(self.interp, op, ins, rows)
            return [produced]
        produced = REGISTRY[op.name](self.interp, op, list(ins), {})
        produced = list(produced) if isinstance(produced, (list, tuple)) else [produced]
        if step.when == ROWS:
            for p in produced:
                if host(p).a.shape[:1] != (rows,):
                    raise NotBlockable(f"{op.name} gave {list(host(p).a.shape)} for a block of {rows} rows")
        return produced


def _gather_rows(interp, op, ins, rows):
    """The gather handler on a block of indices.  The handler shapes its
    result by the op's declared type, so it is handed a stand-in op whose
    result type has the block's leading extent."""
    from types import SimpleNamespace
    ty = op.results[0].type
    block_type = ir.TensorType((rows,) + tuple(ty.shape[1:]), ty.el)
    stand_in = SimpleNamespace(name=op.name, attrs=op.attrs, operands=op.operands, regions=op.regions,
                               results=[SimpleNamespace(type=block_type)])
    return REGISTRY[op.name](interp, stand_in, list(ins), {})


class WeightRows:
    """A match's operand subtrees as `[rows, K]` matrices, whole or in blocks
    of the weight's leading axis (reference qmm.py:1360-1631).

    Blocks are possible when the weight's leading axis is the row axis of the
    `[B * N, K]` matrix (no transpose between the operand and the kernels'
    layout) and whole rows lie inside a block (the groups and the packed
    stream run along K)."""

    def __init__(self, interp, m, args):
        self.interp, self.m, self.args = interp, m, args
        self.arg_number = {a: i for i, a in enumerate(interp._main_block().args)}
        self.lead = m.rshape[0] if m.rshape else 0
        self.step = self._rows_per_block()
        self.tapes = {}
        self.whole = {}

    def _rows_per_block(self):
        m = self.m
        if self.lead < 2 or m.rperm != list(range(len(m.rshape))):
            return None
        per_row = count(m.rshape[1:])
        if per_row <= 0 or per_row % m.K:
            return None
        step = max(1, BLOCK_ELEMS // per_row)
        return step if step < self.lead else None

    def blocked(self) -> bool:
        return self.step is not None

    def unblock(self):
        self.step = None
        self.tapes.clear()

    def blocks(self):
        if self.step is None:
            return [(0, self.lead)]
        return [(lo, min(lo + self.step, self.lead)) for lo in range(0, self.lead, self.step)]

    def forget(self, value):
        """Drop a whole-evaluated operand (it is as large as the weight)."""
        self.whole.pop(value, None)

    def element_type(self, value) -> str:
        return value.type.el

    def rows(self, value, lo, hi):
        if value is None:
            return None
        m = self.m
        if self.step is None:
            got = self.whole.get(value)
            if got is None:
                env = dict(zip(self.interp._main_block().args, self.args))
                got = self.whole[value] = as_rows(evaluate(self.interp, value, env), m)
            return got
        tape = self.tapes.get(value)
        if tape is None:
            tape = self.tapes[value] = _Tape(self.interp, self.args, self.arg_number, self.lead, value)
        a = tape.block(lo, hi)
        for op in m.post:                      # the match's shape ops, on a block
            if op.name == "stablehlo.reshape":
                src, out = dims_of(op.operands[0]), dims_of(op.results[0])
                if (not src or not out or src[0] != self.lead or out[0] != self.lead
                        or count(src[1:]) != count(out[1:])):
                    raise NotBlockable("a reshape below the dot folds the blocked axis")
                a = a.reshape([hi - lo] + out[1:])
            else:
                perm = ir.i64_list(op, "permutation")
                if perm[0] != 0:
                    raise NotBlockable("a transpose below the dot moves the blocked axis")
                a = np.transpose(a, perm)
        if list(a.shape) != [hi - lo] + list(m.rshape[1:]):
            raise NotBlockable(f"a block evaluated to shape {list(a.shape)}")
        return np.ascontiguousarray(a.reshape(-1, m.K))


# ------------------------------------------------------------------ packs ----

def _stamp(buf):
    """What moves when a source buffer is rewritten in place: torch's version
    counter of a tensor (bumped by every in-place write, through any view).
    The reference's buffers are immutable arrays, for which identity says it
    all; a tensor is not.  Host arrays have no such counter (None): they are
    taken as not rewritten, which is the reference's own assumption."""
    try:
        return buf._version
    except (AttributeError, RuntimeError):
        return None


class Pack:
    """The packed arrays of one weight and weak references to the buffers they
    were built from (reference qmm.py:629-664), with each buffer's write stamp
    at that time."""

    def __init__(self, leaves, w, scales, biases, perm, gs, bits, mode="affine"):
        self.sources = [weakref.ref(buf) for buf in leaves]
        self.stamps = [_stamp(buf) for buf in leaves]
        self.w, self.scales, self.biases, self.perm = w, scales, biases, perm
        self.gs, self.bits, self.mode = gs, bits, mode
        self.blocked = False
        self.keepalive = None             # the pack whose arrays this one shares

    def arrays(self):
        """In the order `emit` reads them: w, scales[, biases][, perm]."""
        return [a for a in (self.w, self.scales, self.biases, self.perm) if a is not None]

    def matches(self, leaves) -> bool:
        return len(leaves) == len(self.sources) and all(
            ref() is buf and st == _stamp(buf) for ref, st, buf in zip(self.sources, self.stamps, leaves))

    def alias(self, leaves):
        """The same arrays for another set of source buffers."""
        twin = Pack(leaves, self.w, self.scales, self.biases, self.perm, self.gs, self.bits, self.mode)
        twin.keepalive = self
        twin.blocked = self.blocked
        return twin


def _typed(a: np.ndarray, el: str):
    """Host values in the representation the pack primitives take."""
    if el == "bf16":
        return BF16Array.from_f32(a)
    if el == "f16":
        return np.ascontiguousarray(a, np.float16)
    return np.ascontiguousarray(a)


def _upload(a):
    """Packed arrays live on the GPU when there is one (they are inputs of the
    fused kernel); on a machine without one they stay host arrays, which is
    enough for everything but `emit`."""
    import torch
    if a is None or not torch.cuda.is_available():
        return a
    if isinstance(a, BF16Array):
        return torch.from_numpy(a.bits.view(np.int16).copy()).cuda().view(torch.bfloat16)
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32).copy()).cuda()
    return torch.from_numpy(a.copy()).cuda()


def _stack(parts, m):
    """Row blocks of a packed array back into `[B.., N, last]`."""
    rows = parts[0] if len(parts) == 1 else (
        BF16Array(np.concatenate([p.bits for p in parts], axis=0)) if isinstance(parts[0], BF16Array)
        else np.concatenate(parts, axis=0))
    if m.bshape:
        rows = rows.reshape(tuple(m.bshape) + (m.N, rows.shape[-1]))
    return rows


class _CodeRange:
    """Pass 1 of an affine pack: the width and the offset that make every code
    of the weight an unsigned `bits`-bit number."""

    def __init__(self):
        self.lo = self.hi = None

    def feed(self, codes):
        lo, hi = int(codes.min()), int(codes.max())
        self.lo = lo if self.lo is None else min(self.lo, lo)
        self.hi = hi if self.hi is None else max(self.hi, hi)

    def finish(self):
        span = self.hi - self.lo
        if span >= 256:
            raise Reject(f"the codes run from {self.lo} to {self.hi}: wider than 8 bits")
        bits = 4 if span < 16 else 8
        # signed-code convention first (its bias is a power-of-two multiple of
        # the scale, exact in bf16); otherwise whatever shift makes them fit
        offset = 1 << (bits - 1)
        if self.lo + offset < 0 or self.hi + offset >= (1 << bits):
            offset = -self.lo
        return bits, offset


class _GroupTables:
    """Pass 2 of an affine pack: one scale (and zero point) per group.  Per
    block the maps are checked at the smallest group size and reduced to one
    head per group; the size the whole weight allows is read off the heads."""

    def __init__(self, m, blocked):
        self.m, self.blocked = m, blocked
        self.scale_heads, self.zero_heads = [], []
        self.perm = None

    def feed(self, scale_map, zero_map):
        g0 = packing.GROUP_SIZES[-1]
        maps = [x for x in (scale_map, zero_map) if x is not None]
        if not all(packing.group_const(x, g0) for x in maps):
            if self.blocked:
                # un-interleaving the groups needs the whole contraction axis
                # of the whole weight
                raise NotBlockable(f"scales / zero points vary inside groups of {g0}")
            self.perm = packing.regroup(self.m.K, (scale_map, zero_map))
            if self.perm is not None:
                scale_map = packing.take_k(scale_map, self.perm)
                zero_map = None if zero_map is None else packing.take_k(zero_map, self.perm)
            maps = [x for x in (scale_map, zero_map) if x is not None]
            if not all(packing.group_const(x, g0) for x in maps):
                raise Reject("scales / zero points are not constant over any grouping of K"
                             + (" (columns regrouped)" if self.perm is not None else ""))
        self.scale_heads.append(packing.group_heads(scale_map, g0))
        if zero_map is not None:
            self.zero_heads.append(packing.group_heads(zero_map, g0))

    def finish(self, code_lo, code_hi):
        m, g0 = self.m, packing.GROUP_SIZES[-1]
        scales = np.concatenate(self.scale_heads, axis=0)
        zeros = np.concatenate(self.zero_heads, axis=0) if self.zero_heads else None
        gs = packing.pick_group_heads(m.K, scales, zeros)
        if gs is None:
            raise Reject("no group size makes scales / zero points constant")
        if gs != g0:
            scales = packing.group_heads(scales, gs // g0)
            zeros = None if zeros is None else packing.group_heads(zeros, gs // g0)
        if zeros is not None:
            zeros = zeros.astype(np.float32)
            if not bool((zeros == np.round(zeros)).all()):
                raise Reject("fractional zero points")
            if bool((np.abs(zeros) > 32768).any()):
                raise Reject("zero points beyond +-32768")
            if m.sub_range is not None:
                # the graph subtracts in wrapping integer arithmetic, the
                # fused form exactly: they agree only if nothing can wrap
                low, high = m.sub_range
                if code_lo - int(zeros.max()) < low or code_hi - int(zeros.min()) > high:
                    raise Reject("the graph's integer zero-point subtraction can wrap")
        return scales, zeros, gs


def _per_channel_tables(interp, m, args):
    """Per-channel form: the graph divides the result by a scale per output
    channel; 1 / scale (computed once, in float32) becomes the weight scale of
    every group of that channel, and there are no zero points."""
    env = dict(zip(interp._main_block().args, args))
    sv = evaluate(interp, m.scale, env)
    s = sv.a.astype(np.float32)
    order = sorted(range(len(m.bcast_dims)), key=lambda i: m.bcast_dims[i])
    s = np.transpose(s, order)
    spread = [1] * len(m.nshape)
    for axis, where in enumerate(sorted(m.bcast_dims)):
        spread[where] = s.shape[axis]
    per_channel = np.broadcast_to(s.reshape(spread), m.nshape).reshape(m.N, 1)
    gs = next((g for g in packing.GROUP_SIZES if m.K % g == 0), None)
    if gs is None:
        raise Reject(f"K = {m.K} has no legal group size")
    scales = np.ascontiguousarray(np.broadcast_to(np.float32(1.0) / per_channel, (m.N, m.K // gs)))
    return scales.astype(np.float32), gs, (sv.el if sv.el in ("bf16", "f16") else None)


def build_affine(interp, m, src, args, leaves) -> Pack:
    """Verify and pack a `scale * (codes - zero)` weight."""
    span = _CodeRange()
    for lo, hi in src.blocks():
        span.feed(src.rows(m.codes, lo, hi))
    bits, offset = span.finish()
    perm = zeros = None
    if m.recip:
        scales, gs, table_kind = _per_channel_tables(interp, m, args)
    else:
        tables = _GroupTables(m, src.blocked())
        for lo, hi in src.blocks():
            tables.feed(src.rows(m.scale, lo, hi), src.rows(m.zero, lo, hi))
            src.forget(m.scale)
            src.forget(m.zero)
        scales, zeros, gs = tables.finish(span.lo, span.hi)
        perm = tables.perm
        el = src.element_type(m.scale)
        table_kind = el if el in ("bf16", "f16") else None
    words = []
    for lo, hi in src.blocks():
        codes = src.rows(m.codes, lo, hi).astype(np.int64)
        if perm is not None:
            codes = packing.take_k(codes, perm)
        words.append(packing.pack_codes((codes + offset).astype(np.uint8), bits))
        src.forget(m.codes)
    scales, biases = packing.scale_bias(scales, zeros, offset, table_kind)
    return share(leaves, _stack(words, m), _stack([scales], m), _stack([biases], m), perm, gs, bits,
                 "affine")


def build_mxfp4(interp, m, src, args, leaves) -> Pack:
    """Verify and pack an MXFP4 weight: every value must sit on the E2M1 grid
    of its type, every scale must be one power of two per 32 values."""
    gs = packing.MXFP4_GROUP
    if m.K % gs:
        raise Reject(f"K = {m.K} is not a multiple of {gs}")
    perm = None
    words, scale_bytes = [], []
    for lo, hi in src.blocks():
        scale_map = src.rows(m.scale, lo, hi)
        if not packing.group_const(scale_map, gs):
            if src.blocked():
                raise NotBlockable(f"MXFP4 scales vary inside groups of {gs}")
            perm = packing.regroup(m.K, (scale_map,))
            if perm is not None:
                scale_map = packing.take_k(scale_map, perm)
            if not packing.group_const(scale_map, gs):
                raise Reject(f"MXFP4 scales are not constant over groups of {gs}")
        scale_bytes.append(packing.mxfp4_scale_bytes(packing.group_heads(scale_map, gs)))
        src.forget(m.scale)
        values = _typed(src.rows(m.codes, lo, hi), src.element_type(m.codes))
        if perm is not None:
            values = packing.take_k(values, perm)
        words.append(packing.pack_codes(packing.mxfp4_codes(values), 4))
        src.forget(m.codes)
    return share(leaves, _stack(words, m), _stack(scale_bytes, m), None, perm, gs, 4, "mxfp4")


def build(interp, m, args, leaves) -> Pack:
    """One match's weight, verified and packed on concrete buffers: by row
    blocks when the subtree allows it, else from a whole evaluation."""
    src = WeightRows(interp, m, args)
    builder = build_mxfp4 if m.mode == "mxfp4" else build_affine
    while True:
        try:
            pk = builder(interp, m, src, args, leaves)
            break
        except NotBlockable as why:
            if not src.blocked():
                raise Reject(str(why)) from None
            _debug(f"{m.name} packs from a whole evaluation ({why})")
            src.unblock()
    pk.blocked = src.blocked()
    STATS["blocked"] += int(pk.blocked)
    STATS["packs"] += 1
    STATS["perms"] += int(pk.perm is not None)
    STATS["mxfp4"] += int(pk.mode == "mxfp4")
    STATS["batched"] += int(bool(m.bshape))
    _debug(f"packed {m.name} mode={pk.mode} bits={pk.bits} group={pk.gs}"
           f"{' regrouped' if pk.perm is not None else ''}{' by blocks' if pk.blocked else ''}")
    for buf in leaves:                   # a pack is keyed by buffer identity: the buffers must not change under it
        freeze(buf)
    return pk


def freeze(buf):
    """Host storage a pack was built from is made read-only (an in-place
    update would otherwise keep serving the stale pack)."""
    a = getattr(buf, "a", None)
    if isinstance(a, np.ndarray):
        try:
            a.flags.writeable = False
        except ValueError:
            pass


# ---- content-addressed sharing (tied or duplicated weights) ---------------
_SHARED = {}


def _digest(arrays) -> str:
    h = hashlib.blake2b(digest_size=16)
    for a in arrays:
        if a is None:
            h.update(b"-")
            continue
        b = np.ascontiguousarray(a.bits if isinstance(a, BF16Array) else a)
        h.update(str((isinstance(a, BF16Array), b.dtype.str, b.shape)).encode())
        h.update(b.tobytes())
    return h.hexdigest()


def share(leaves, w, scales, biases, perm, gs, bits, mode) -> Pack:
    """Host-packed arrays -> a pack holding device arrays.  A pack whose bytes
    equal those of a live earlier pack shares that pack's arrays instead of
    uploading a copy (reference qmm.py:1656-1704)."""
    perm = None if perm is None else np.ascontiguousarray(perm, np.int32)
    key = (mode, gs, bits, _digest([w, scales, biases, perm])) if MAX_SHARED > 0 else None
    if key is not None:
        ref = _SHARED.get(key)
        earlier = ref() if ref is not None else None
        if earlier is not None:
            STATS["shared"] += 1
            return earlier.alias(leaves)
    pk = Pack(leaves, _upload(w), _upload(scales), _upload(biases), _upload(perm), gs, bits, mode)
    if key is not None:
        if len(_SHARED) >= MAX_SHARED:
            for dead in [k for k, ref in _SHARED.items() if ref() is None]:
                del _SHARED[dead]
            if len(_SHARED) >= MAX_SHARED:
                _SHARED.clear()
        _SHARED[key] = weakref.ref(pk)
    return pk


# ---- cross-executable build cache: (canonical text of the reconstruction
# subtree, identity of the buffers it reads) -> pack
_BUILT = {}


def _canon_callee(name, module, stack):
    """A private function as text that does not depend on names: its body in
    program order, values by position."""
    name = str(name).lstrip("@")
    if module is None or name not in module.funcs:
        raise Reject("callee not found")
    if name in stack:
        raise Reject("recursive callee")

    def closed(v):
        raise Reject("a function body reads a value from outside")
    return _canon_block(module.funcs[name].body, module, closed, stack + (name,))


def _canon_block(block, module, outer, stack):
    ids = {a: f"b{i}:{a.type}" for i, a in enumerate(block.args)}

    def look(v):
        return ids[v] if v in ids else outer(v)
    lines = []
    for n, o in enumerate(block.ops):
        lines.append(_canon_op(o, n, [look(x) for x in o.operands], module, look, stack))
        for i, r in enumerate(o.results):
            ids[r] = f"%{n}.{i}"
    return ";".join(lines)


# A constant of more than this many elements is a weight baked into the
# program: serializing it costs more than the build the cache would save, so
# such a chain is built every time (reference qmm.py:1965-1975); the same for
# any attribute whose printed form is very long.
FP_DENSE_ELEMS = 1024
FP_ATTR_CHARS = 1 << 16


def _canon_op(o, n, opnds, module, look, stack):
    """One op of a canonical text: name, attributes, what it calls and the
    regions it holds by *content* (a callee's name is not part of the key, its
    body is: two programs that differ in the name are the same chain, two that
    differ in the body are not), operands, result types."""
    attrs = dict(o.attrs)
    if o.name == "stablehlo.constant" and o.results:
        shape = getattr(o.results[0].type, "shape", None)
        if shape is not None and int(np.prod(shape, dtype=np.int64)) > FP_DENSE_ELEMS:
            raise Reject(f"a constant of {int(np.prod(shape, dtype=np.int64))} elements")
    called = ""
    for ref in ("callee", "decomposition"):
        if ref in attrs and (o.name == "func.call" or ref == "decomposition"):
            called += "{" + _canon_callee(attrs.pop(ref), module, stack) + "}"
    regions = "".join("{" + _canon_block(r, module, look, stack) + "}" for r in o.regions)
    shown = sorted((k, repr(val)) for k, val in attrs.items())
    if any(len(text) > FP_ATTR_CHARS for _, text in shown):
        raise Reject("an attribute too long to serialize")
    return f"{n}={o.name}{shown}{called}{regions}({','.join(opnds)})->{[str(r.type) for r in o.results]}"


def fingerprint(m, module=None):
    """Canonical serialization of the reconstruction subtree: ops in a
    deterministic post-order, operands by position, leaves by argument slot,
    callees and regions by their bodies (reference qmm.py:2022-2268 keeps the
    same two-part key)."""
    if m.fp is not None:
        return m.fp
    ids, lines = {}, []
    arg_slot = {}

    def visit(v):
        v = outer_definition(v) if v.is_block_arg else v
        if v in ids:
            return ids[v]
        if v.is_block_arg:
            slot = arg_slot.setdefault(v, len(arg_slot))
            ids[v] = f"a{slot}:{v.type}"
            return ids[v]
        o = v.op
        if o.name in OPAQUE_OPS:
            raise Reject("opaque op in subtree")
        opnds = [visit(x) for x in o.operands]
        n = len(lines)
        lines.append(_canon_op(o, n, opnds, module, visit, ()))
        for i, r in enumerate(o.results):
            ids[r] = f"%{n}.{i}"
        return ids[v]

    try:
        parts = [visit(x) for x in (m.codes, m.zero, m.scale) if x is not None]
        extra = (m.mode, m.recip, m.rperm, m.rshape, m.bcast_dims,
                 [(o.name, repr(sorted(o.attrs.items(), key=str))) for o in m.post])
        m.fp = ("\n".join(lines) + "|" + ",".join(parts) + "|" + repr(extra),
                [a.index for a in sorted(arg_slot, key=arg_slot.get)])
    except (Reject, RecursionError):
        m.fp = False
        STATS["build_declines"] += 1
    return m.fp


def _build_key(m, args, module=None):
    if MAX_BUILT <= 0:
        return None, None
    fp = fingerprint(m, module)
    if not fp:
        return None, None
    text, slots = fp
    keyleaves = [args[i] for i in slots]
    return (text, tuple(id(a) for a in keyleaves)), keyleaves


def _cached_build(key, keyleaves):
    hit = _BUILT.get(key)
    if hit is None:
        return None
    refs, stamps, pref = hit
    pk = pref()
    if pk is None or len(refs) != len(keyleaves) or not all(
            r() is a and st == _stamp(a) for r, st, a in zip(refs, stamps, keyleaves)):
        _BUILT.pop(key, None)
        return None
    return pk


def _remember_build(key, keyleaves, pk):
    if len(_BUILT) >= MAX_BUILT:
        for dead in [k for k, (refs, _, pref) in _BUILT.items()
                     if pref() is None or any(r() is None for r in refs)]:
            del _BUILT[dead]
        if len(_BUILT) >= MAX_BUILT:
            _BUILT.clear()
    _BUILT[key] = ([weakref.ref(a) for a in keyleaves], [_stamp(a) for a in keyleaves], weakref.ref(pk))


def pack_for(interp, m, args, check=lambda m: None):
    """The pack of match `m` for these argument buffers: one the match already
    holds for exactly these buffers (most recent first), else one another
    executable built from the same subtree and buffers, else a fresh build
    (reference qmm.py:2271-2302).  `check(m)` runs before a fresh build and
    may Reject what the kernels do not serve."""
    leaves = [args[i] for i in m.arg_indices]
    for age, held in enumerate(m.packs):
        if held.matches(leaves):
            if age:
                m.packs.insert(0, m.packs.pop(age))
            return held

    def adopt(pk):
        m.packs.insert(0, pk)
        del m.packs[MAX_PACKS:]
        return pk

    key, keyleaves = _build_key(m, args, getattr(interp, "module", None))
    if key is not None:
        elsewhere = _cached_build(key, keyleaves)
        if elsewhere is not None:
            STATS["build_hits"] += 1
            return adopt(elsewhere.alias(leaves))
    m.repacks += 1
    if m.repacks > MAX_REPACKS:
        raise Reject(f"the weight's buffers changed {m.repacks} times: repacking costs more than "
                     "the chain it replaces")
    check(m)
    pk = build(interp, m, args, leaves)
    if key is not None:
        _remember_build(key, keyleaves, pk)
    return adopt(pk)
