"""Structural half of the quantized-matmul recognizer: which dots of a program
read a weight that is rebuilt, inside the graph, from integer codes.

The job and the accepted graph shapes are those of the reference's matcher
(reference src/metaljax/qmm.py:509-1091); the formulation is this package's
own, over the SSA graph of `metaljax_amd.ir`:

  * an operand is looked at through a `View`: the value at the bottom of a
    run of pass-through ops (reshape / transpose / convert / broadcast) plus
    the run itself, so every pattern is a few questions asked of views;
  * a dot's loop structure is a `DotShape` (batch / free / contracting axes of
    both sides, and the [B, M, K] x [B, N, K] sizes they fold to);
  * a pattern yields a `Match`: the three operand subtrees (codes, zero point,
    scale) that the pack step evaluates once, the ops the rewrite absorbs, and
    the loop structure;
  * `settle` decides which absorbed ops can really be skipped by marking what
    must still run (an op with a consumer outside the rewrite, and everything
    such an op reads) and drops candidates whose own reconstruction is among
    them.

Nothing here looks at values.  Three graph shapes are recognized, on either
operand of a dot (a weight on the left gives a transposed result):

  sub-channel   dot(x, shape-ops(multiply(convert(codes) [- zero], scales)))
  per-channel   divide(dot(x, convert(codes)), broadcast(scale))
  MXFP4         dot(x, shape-ops(multiply(values, broadcast(one scale per 32))))
"""

from __future__ import annotations

import os
from dataclasses import dataclass, field

from . import ir
from .interpreter import FLOAT_ELS
from .packing import GROUP_SIZES, MXFP4_GROUP, Reject

BATCHED_DOTS = os.environ.get("METALJAX_QMM_BATCH", "1") != "0"

INT_ELS = frozenset({"i4", "ui4", "i8", "i16", "i32", "i64", "ui8", "ui16", "ui32", "ui64"})
SHAPE_OPS = frozenset({"stablehlo.reshape", "stablehlo.transpose"})
# ops whose result cannot be recomputed from the operands alone
OPAQUE_OPS = frozenset({"stablehlo.while", "stablehlo.if", "stablehlo.case", "stablehlo.custom_call",
                        "stablehlo.optimization_barrier"})
_SIGNED_BITS = {"i4": 4, "i8": 8, "i16": 16, "i32": 32, "i64": 64}
_ACTIVATION_ELS = frozenset({"bf16", "f16", "f32"})      # what the kernels multiply (f64 dots stay literal)


def elem(v) -> str:
    return v.type.el


def dims_of(v) -> list:
    return list(v.type.shape)


def count(extents) -> int:
    n = 1
    for e in extents:
        n *= e
    return n


def op_key(op):
    """An operation is named by its first result (None for ops without one)."""
    return op.results[0] if op.results else None


# ----------------------------------------------------------------- views ----

@dataclass
class View:
    """`base` seen through `through` (ops listed from `base` outwards)."""
    base: object
    through: list

    def shape_ops(self):
        return [o for o in self.through if o.name in SHAPE_OPS]


def look_through(v, kinds) -> View:
    """Descend from `v` while its producer is one of `kinds` (unary ops)."""
    run = []
    while v.op is not None and v.op.name in kinds:
        run.append(v.op)
        v = v.op.operands[0]
    run.reverse()
    return View(v, run)


_CONVERT = frozenset({"stablehlo.convert"})
_SHAPE_OR_CONVERT = SHAPE_OPS | _CONVERT


def broadcast_source(v):
    """If `v` is (converts of) a chain of broadcast_in_dim ops: the value that
    is broadcast and, for each of its axes, the axis of `v` it ends up on;
    (v, None) when no broadcast is involved (reference qmm.py:563-585)."""
    placement = list(range(len(dims_of(v))))
    found = False
    while v.op is not None:
        name = v.op.name
        if name == "stablehlo.broadcast_in_dim":
            inner = ir.i64_list(v.op, "broadcast_dimensions")
            placement = [placement[axis] for axis in inner]
            found = True
        elif name != "stablehlo.convert":
            break
        v = v.op.operands[0]
    return v, (placement if found else None)


def outer_definition(v):
    """A while-loop argument that the loop only carries around (the body hands
    argument i back as result i) stands for what the loop was started with:
    climb out of such loops, at most eight deep (reference qmm.py:714-740)."""
    for _ in range(8):
        if not v.is_block_arg:
            break
        loop = v.block.parent_op
        if loop is None or loop.name != "stablehlo.while":
            break
        cond, body = loop.regions[0], loop.regions[1]
        if v.block is not body and v.block is not cond:
            break
        if body.terminator.operands[v.index] is not body.args[v.index]:
            break                                   # the loop changes it
        v = loop.operands[v.index]
    return v


# ---------------------------------------------------------------- a match ----

@dataclass(eq=False)
class Match:
    """One recognized quantized matmul.  Field names follow the reference's
    record (reference qmm.py:588-626): other modules and the tests read them."""
    # the rewrite: `root` (named by `key`) is replaced, `ops` are skipped,
    # `required` are the skipped ops without which the rewrite makes no sense
    root: object = None
    key: object = None
    ops: dict = field(default_factory=dict)
    required: list = field(default_factory=list)
    absorbed: bool = False            # taken over by an expert dispatch: no dense product is emitted
    disabled: bool = False
    # operand subtrees, evaluated once at pack time
    lhs: object = None                # the activation operand, read at every step
    codes: object = None
    zero: object = None
    scale: object = None
    sub_range: tuple = None           # value range of an INTEGER codes - zero, None for a float one
    recip: bool = False               # per-channel form: the scale divides the result
    bcast_dims: list = None           # per-channel form: where the divisor's axes land among the N axes
    post: list = field(default_factory=list)      # shape ops between the multiply and the dot
    mode: str = "affine"
    arg_indices: tuple = ()           # @main arguments the subtrees read
    # loop structure: operand axis orders that give [B, M, K] and [B, N, K]
    lperm: list = None
    rperm: list = None
    rshape: list = None
    bshape: list = field(default_factory=list)
    mshape: list = field(default_factory=list)
    nshape: list = field(default_factory=list)
    B: int = 1
    M: int = 0
    K: int = 0
    N: int = 0
    swapped: bool = False             # the weight is the dot's left operand
    out_dtype: str = "bf16"
    act_dtype: str = "bf16"
    name: str = "?"
    # pack state (filled at the first execute)
    packs: list = field(default_factory=list)
    repacks: int = 0
    slot: int = -1
    nvals: int = 0
    gs: int = 0
    bits: int = 0
    has_perm: bool = False
    fp: object = None                 # build-cache fingerprint (None: not computed, False: declined)


@dataclass
class DotShape:
    """Axis roles of a dot_general with the quantized operand on side `qside`."""
    act_batch: list
    act_free: list
    act_contract: list
    q_batch: list
    q_free: list
    q_contract: list

    @classmethod
    def of(cls, dot, qside):
        lb, rb, lc, rc = ir.dot_dims(dot)
        q, a = ((rb, rc), (lb, lc)) if qside == 1 else ((lb, lc), (rb, rc))
        arank = len(dims_of(dot.operands[1 - qside]))
        qrank = len(dims_of(dot.operands[qside]))
        return cls(act_batch=list(a[0]), act_contract=list(a[1]),
                   act_free=[d for d in range(arank) if d not in a[0] and d not in a[1]],
                   q_batch=list(q[0]), q_contract=list(q[1]),
                   q_free=[d for d in range(qrank) if d not in q[0] and d not in q[1]])


class Program:
    """What the patterns need to know about the enclosing program."""

    def __init__(self, interp):
        main = interp._main_block()
        self.arg_number = {a: i for i, a in enumerate(main.args)}
        self.donated = frozenset(interp.donated_args)
        self.main = main


def collect_subtree(prog, outputs, absorbed, always=()):
    """Every op that `outputs` are computed from, down to @main's arguments
    (whose numbers are returned) and constants, into `absorbed`; loop carries
    are followed outwards.  `always`: ops absorbed whatever they feed."""
    for o in always:
        absorbed[op_key(o)] = o
    reads = set()
    todo, done = list(outputs), set()
    while todo:
        v = todo.pop()
        if v in done:
            continue
        done.add(v)
        if not v.is_block_arg:
            producer = v.op
            if producer.name in OPAQUE_OPS:
                raise Reject(f"the weight is computed through {producer.name}")
            absorbed.setdefault(op_key(producer), producer)
            todo.extend(producer.operands)
            continue
        number = prog.arg_number.get(v)
        if number is not None:
            reads.add(number)
            continue
        outside = outer_definition(v)
        if outside is v:
            raise Reject("the weight depends on a value produced inside a loop or branch")
        todo.append(outside)
    return reads


def fill_geometry(prog, m, root, dot, qside, absorb, required=(), always=()):
    """Loop structure, types and the absorbed subtree of a candidate whose
    quantized operand is operand `qside` of `dot` (reference qmm.py:780-841)."""
    ds = DotShape.of(dot, qside)
    if (ds.q_batch or ds.act_batch) and not BATCHED_DOTS:
        raise Reject("batched dot (METALJAX_QMM_BATCH=0)")
    weight, act = dot.operands[qside], dot.operands[1 - qside]
    if elem(act) not in _ACTIVATION_ELS:
        raise Reject(f"activations of type {elem(act)}")
    result_el = elem(root.results[0])
    if result_el not in _ACTIVATION_ELS:
        raise Reject(f"result of type {result_el}")
    wdims, adims = dims_of(weight), dims_of(act)
    if [adims[d] for d in ds.act_batch] != [wdims[d] for d in ds.q_batch]:
        raise Reject("batch extents differ between the operands")
    m.bshape = [adims[d] for d in ds.act_batch]
    m.mshape = [adims[d] for d in ds.act_free]
    m.nshape = [wdims[d] for d in ds.q_free]
    m.B, m.M, m.N = count(m.bshape), count(m.mshape), count(m.nshape)
    m.K = count(adims[d] for d in ds.act_contract)
    if 0 in (m.B, m.M, m.N, m.K):
        raise Reject("empty product")
    if m.K != count(wdims[d] for d in ds.q_contract):
        raise Reject("contracted extents differ between the operands")
    smallest = GROUP_SIZES[-1]
    if m.K % smallest:
        raise Reject(f"K = {m.K} is not a multiple of {smallest}")
    m.root, m.key, m.lhs = root, op_key(root), act
    m.swapped = qside == 0
    m.lperm = ds.act_batch + ds.act_free + ds.act_contract
    m.rperm = ds.q_batch + ds.q_free + ds.q_contract
    m.rshape = wdims
    m.out_dtype, m.act_dtype = result_el, elem(act)
    sizes = f"{m.M}x{m.K}x{m.N}"
    if m.bshape:
        sizes = "x".join(str(e) for e in m.bshape) + "|" + sizes
    m.name = sizes + ("'" if m.swapped else "")
    reads = collect_subtree(prog, absorb, m.ops, always)
    if reads & prog.donated:
        raise Reject("the weight is read from a donated argument, which the program may overwrite")
    m.arg_indices = tuple(sorted(reads))
    m.required = [op_key(o) for o in required] + [op_key(o) for o in m.post]
    return m


# ------------------------------------------------------------- patterns ----

def integer_codes(v):
    """`v` as (convert of) integer codes, optionally minus a zero point:
    (codes, zero or None, range of an integer subtraction or None); None when
    `v` is neither (reference qmm.py:531-555).  An integer `codes - zero`
    wraps in the graph but not in the fused form, hence the range."""
    below = look_through(v, _CONVERT).base
    producer = below.op
    if producer is not None and producer.name == "stablehlo.subtract":
        minuend = look_through(producer.operands[0], _CONVERT).base
        if elem(minuend) not in INT_ELS:
            return None
        span = None
        if elem(below) in INT_ELS:                  # subtracted as integers
            width = _SIGNED_BITS.get(elem(below))
            if width is None:
                return None                         # unsigned subtraction: modular by design
            span = (-(1 << (width - 1)), (1 << (width - 1)) - 1)
        return minuend, producer.operands[1], span
    if elem(below) in INT_ELS:
        return below, None, None
    return None


def reads_integers(v, budget=64) -> bool:
    """Is an integer-typed value among the first `budget` values below `v`?"""
    todo, done = [v], set()
    while todo and len(done) < budget:
        cur = todo.pop()
        if cur in done:
            continue
        done.add(cur)
        if elem(cur) in INT_ELS:
            return True
        if cur.op is not None and cur.op.name not in OPAQUE_OPS:
            todo.extend(cur.op.operands)
    return False


def block_scaled_factors(mul):
    """The two factors of an MXFP4 reconstruction `values * scale`, told apart
    by shape alone: the scale is the factor that is a broadcast of exactly one
    element per 32 of the product (reference qmm.py:868-899)."""
    product = count(dims_of(mul.results[0]))
    scale_sides = []
    for side, factor in enumerate(mul.operands):
        if elem(factor) not in FLOAT_ELS:
            raise Reject(f"a factor of type {elem(factor)}")
        source, placement = broadcast_source(factor)
        if placement is None:
            continue
        entries = count(dims_of(source))
        if entries and entries * MXFP4_GROUP == product:
            scale_sides.append(side)
    if len(scale_sides) != 1:
        why = ("no factor is one scale per %d values" % MXFP4_GROUP if not scale_sides
               else "both factors look like block scales")
        raise Reject(why)
    side = scale_sides[0]
    return mul.operands[1 - side], mul.operands[side]


def scaled_weight(prog, dot, qside):
    """Sub-channel affine and MXFP4: the operand is shape-ops of a multiply."""
    operand = dot.operands[qside]
    seen = look_through(operand, _SHAPE_OR_CONVERT)
    mul = seen.base.op
    if mul is None or mul.name != "stablehlo.multiply":
        raise Reject("the operand is not a product")
    m = Match(post=seen.shape_ops())
    for side in (0, 1):
        found = integer_codes(mul.operands[side])
        if found is not None:
            m.codes, m.zero, m.sub_range = found
            m.scale = mul.operands[1 - side]
            break
    else:
        values, m.scale = block_scaled_factors(mul)
        if not reads_integers(values):
            raise Reject("no integer codes under the scaled values")
        m.mode, m.codes = "mxfp4", values
    if elem(m.scale) not in FLOAT_ELS:
        raise Reject(f"scales of type {elem(m.scale)}")
    return fill_geometry(prog, m, dot, dot, qside, absorb=[operand], required=[mul])


def scaled_weight_either_side(prog, dot):
    first_reason = None
    for qside in (1, 0):                              # the common layout first
        try:
            return scaled_weight(prog, dot, qside)
        except Reject as why:
            first_reason = first_reason or why
    raise first_reason


def per_channel_weight(prog, div):
    """Symmetric per-channel: the dot multiplies raw integer codes and its
    result is divided by a per-output-channel scale."""
    numerator, divisor = div.operands
    dot = numerator.op
    if dot is None or dot.name != "stablehlo.dot_general":
        raise Reject("the dividend is not a dot")
    seen = look_through(dot.operands[1], _SHAPE_OR_CONVERT)
    if elem(seen.base) not in INT_ELS:
        raise Reject("the dot's right operand is not integer codes")
    scale, placement = broadcast_source(divisor)
    if placement is None:
        raise Reject("the divisor is not a broadcast")
    if elem(scale) not in FLOAT_ELS:
        raise Reject(f"a divisor of type {elem(scale)}")
    lb, rb, lc, _ = ir.dot_dims(dot)
    if lb or rb:
        raise Reject("batched dot under a per-channel divide")
    row_axes = len(dims_of(dot.operands[0])) - len(lc)        # leading result axes that index activation rows
    if any(axis < row_axes for axis in placement):
        raise Reject("the divisor varies along the activation rows")
    m = Match(recip=True, codes=seen.base, scale=scale, post=seen.shape_ops(),
              bcast_dims=[axis - row_axes for axis in placement])
    return fill_geometry(prog, m, div, dot, 1, absorb=[dot.operands[1], divisor],
                         required=[dot], always=[dot])


# ----------------------------------------------------- what may be skipped ----

def settle(candidates, note=lambda text: None):
    """An absorbed op can be skipped only if nothing outside the rewrite reads
    it.  Mark what must still run -- an absorbed op with a reader that is
    neither absorbed nor a rewritten root, and (since it then runs) every
    absorbed op it reads, transitively -- and drop the candidates whose own
    `required` ops are marked; dropping one changes the picture, so repeat
    until nothing is dropped (reference qmm.py:991-1039)."""
    alive = list(candidates)
    while alive:
        pool = {}
        for m in alive:
            pool.update(m.ops)
        rewritten = {m.key for m in alive}
        must_run, frontier = set(), []
        for key, op in pool.items():
            readers = (op_key(user) for res in op.results for user in res.uses)
            if any(r is None or (r not in pool and r not in rewritten) for r in readers):
                frontier.append(key)
        while frontier:
            key = frontier.pop()
            if key in must_run:
                continue
            must_run.add(key)
            for operand in pool[key].operands:
                if operand.op is not None and op_key(operand.op) in pool:
                    frontier.append(op_key(operand.op))
        losers = [m for m in alive if any(k in must_run for k in m.required)]
        if not losers:
            for m in alive:
                m.ops = {k: o for k, o in m.ops.items() if k not in must_run}
            break
        for m in losers:
            note(f"dropped {m.name} (its reconstruction is read elsewhere too)")
        alive = [m for m in alive if m not in losers]
    return alive


def find_matches(interp, note=lambda text: None):
    """Every quantized matmul of the program, settled."""
    prog = Program(interp)
    found = []
    for block in ir.walk_blocks(prog.main):
        for op in block.ops:
            pattern = _PATTERNS.get(op.name)
            if pattern is None:
                continue
            try:
                found.append(pattern(prog, op))
            except Reject:
                continue
    # a dot that is itself inside another candidate's absorbed subtree (the
    # dot under a per-channel divide) is not a candidate of its own
    inside = set()
    for m in found:
        inside.update(m.ops)
    return settle([m for m in found if m.key not in inside], note)


_PATTERNS = {"stablehlo.dot_general": scaled_weight_either_side,
             "stablehlo.divide": per_channel_weight}
