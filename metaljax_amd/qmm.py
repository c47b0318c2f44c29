"""Recognizer that maps dequantize-then-matmul chains onto one fused quantized
matmul served by the gfx950 HIP kernels.

Same job, entry points and failure behaviour as the reference recognizer
(reference src/metaljax/qmm.py): `analyze` finds the chains structurally,
`prologue` verifies and packs each weight once against concrete buffers,
`emit` replaces the whole chain at run time.  Three forms are recognized:

  sub-channel / asymmetric   dot(x, [reshape/transpose](mul(sub(cvt(codes), cvt(zeros)), scales)))
  per-channel / symmetric    divide(dot(x, cvt(codes)), broadcast(scale))
  MXFP4                      dot(x, [reshape](mul(decode(codes), broadcast(2**(e8m0-127)))))

on either operand of the dot (a weight on the left gives a transposed
result).  The ops between the integer codes and the multiply are not matched
one by one: the three operand subtrees are recorded and evaluated once, on the
host, at the first execute; every value-level question (codes fit 4 or 8
bits, maps constant per group, integer zero points, E2M1 grid membership,
power-of-two scales) is answered there, and any failure disables that one dot,
which then runs literally.

What differs from the reference is below the boundary: the fused op is
`metaljax_amd.kernels.quantized_matmul` (libqmm_hip.so through ctypes) on
device tensors, and packing runs in numpy on the host.  A missing library or
GPU is an error at `emit`, never a silent literal run.
"""

from __future__ import annotations

import hashlib
import os
import weakref
from collections import deque

import numpy as np

from . import ir, packing
from .interpreter import FLOAT_ELS, HostArray, REGISTRY, host
from .packing import BF16Array, Reject

QMM_ENABLED = os.environ.get("METALJAX_QMM", "1") != "0"
ENABLED = QMM_ENABLED or os.environ.get("METALJAX_MOE", "1") != "0"
_DEBUG = os.environ.get("METALJAX_DEBUG", "") == "1"
_GROUP_SIZES = packing.GROUP_SIZES
_MAX_PACKS = int(os.environ.get("METALJAX_QMM_CACHE", "2"))
_MAX_REPACKS = int(os.environ.get("METALJAX_QMM_REPACKS", "8"))
_BATCH = os.environ.get("METALJAX_QMM_BATCH", "1") != "0"
_SHARE = os.environ.get("METALJAX_QMM_SHARE", "1") != "0"
_BUILD_CACHE = os.environ.get("METALJAX_QMM_BUILD_CACHE", "1") != "0"
_MXFP4_GROUP = packing.MXFP4_GROUP

# Diagnostics (tests assert on these; nothing else reads them).
STATS = {"recognized": 0, "packs": 0, "fallbacks": 0, "perms": 0, "mxfp4": 0, "batched": 0,
         "shared": 0, "blocked": 0, "build_hits": 0, "build_declines": 0}


def stats() -> dict:
    return dict(STATS)


def reset_stats():
    for k in STATS:
        STATS[k] = 0


_INT_ELS = {"i4", "ui4", "i8", "i16", "i32", "i64", "ui8", "ui16", "ui32", "ui64"}
_SHAPE_OPS = ("stablehlo.reshape", "stablehlo.transpose")
_OPAQUE = ("stablehlo.while", "stablehlo.if", "stablehlo.case", "stablehlo.custom_call",
           "stablehlo.optimization_barrier")
_SIGNED_WIDTH = {"i4": 4, "i8": 8, "i16": 16, "i32": 32, "i64": 64}
_Reject = Reject


def _debug(msg):
    if _DEBUG:
        print(f"[metaljax_amd] qmm: {msg}", flush=True)


# --------------------------------------------------------------------------
# structural matching
# --------------------------------------------------------------------------

def _el(v) -> str:
    return v.type.el


def _is_int(v) -> bool:
    return _el(v) in _INT_ELS


def _shape(v):
    return list(v.type.shape)


def _prod(xs) -> int:
    p = 1
    for x in xs:
        p *= x
    return p


def _key(op):
    """Identity key of an operation: its first result."""
    return op.results[0] if op.results else None


def _strip(v, names):
    """Walk down through `names`-kind ops: (base, ops outermost-last)."""
    chain = []
    while v.op is not None and v.op.name in names:
        chain.append(v.op)
        v = v.op.operands[0]
    return v, list(reversed(chain))


def _strip_shape(v):
    return _strip(v, _SHAPE_OPS + ("stablehlo.convert",))


def _strip_converts(v):
    return _strip(v, ("stablehlo.convert",))


def _parse_codes(v):
    """`v` as an integer-code operand: (codes, zero_point, subtract_range).
    subtract_range is the (lo, hi) an INTEGER `codes - zero` is computed in
    (the fused form evaluates it exactly, so a graph that could wrap must not
    be rewritten); None for a floating-point subtraction.
    (reference src/metaljax/qmm.py:531-555)"""
    base, _ = _strip_converts(v)
    o = base.op
    if o is not None and o.name == "stablehlo.subtract":
        c, _ = _strip_converts(o.operands[0])
        if not _is_int(c):
            return None
        rng = None
        if _is_int(base):
            w = _SIGNED_WIDTH.get(_el(base))
            if w is None:
                return None
            rng = (-(1 << (w - 1)), (1 << (w - 1)) - 1)
        return c, o.operands[1], rng
    if _is_int(base):
        return base, None, None
    return None


def _bcast_chain(v):
    """Peel broadcast_in_dim (and convert) ops: (base, dims) where dims[i] is
    the dimension of `v` that base's dimension i lands in; dims is None when
    the head is not a broadcast (reference qmm.py:563-585)."""
    dims = list(range(len(_shape(v))))
    base = None
    while v.op is not None:
        o = v.op
        if o.name == "stablehlo.broadcast_in_dim":
            d = ir.i64_list(o, "broadcast_dimensions")
            dims = [dims[j] for j in d]
            v = o.operands[0]
            base = v
        elif o.name == "stablehlo.convert":
            v = o.operands[0]
        else:
            break
    return (v, dims) if base is not None else (v, None)


class Match:
    """One recognized quantized matmul (reference qmm.py:588-626)."""

    def __init__(self):
        self.root = self.key = self.lhs = self.codes = self.scale = None
        self.recip = False
        self.fp = None
        self.absorbed = False
        self.mode = "affine"
        self.zero = None
        self.sub_range = None
        self.post = []
        self.bcast_dims = None
        self.ops = {}
        self.required = []
        self.arg_indices = ()
        self.disabled = False
        self.slot = -1
        self.nvals = 0
        self.gs = 0
        self.bits = 0
        self.has_perm = False
        self.packs = []
        self.repacks = 0
        self.name = "?"
        self.lperm = self.rperm = self.rshape = None
        self.bshape, self.mshape, self.nshape = [], [], []
        self.B, self.M, self.K, self.N = 1, 0, 0, 0
        self.out_dtype = "bf16"
        self.act_dtype = "bf16"
        self.swapped = False


class _Pack:
    """Packed arrays of one weight + weak references to the source buffers
    they were built from (reference qmm.py:629-664)."""

    def __init__(self, leaves, w, scales, biases, perm, gs, bits, mode="affine"):
        self.refs = [weakref.ref(a) for a in leaves]
        self.w, self.scales, self.biases = w, scales, biases
        self.perm = perm
        self.gs, self.bits = gs, bits
        self.mode = mode
        self.blocked = False

    def arrays(self):
        out = [self.w, self.scales]
        if self.biases is not None:
            out.append(self.biases)
        if self.perm is not None:
            out.append(self.perm)
        return out

    def matches(self, leaves) -> bool:
        if len(leaves) != len(self.refs):
            return False
        return all(r() is a for r, a in zip(self.refs, leaves))


class State:
    """Per-program recognizer state (reference qmm.py:667-699)."""

    def __init__(self):
        self.matches = []
        self.moe = []
        self.skip = frozenset()
        self.roots = {}
        self.values = []
        self.active = False

    def rebuild(self):
        live = [m for m in self.matches if not m.disabled]
        self.roots = {m.key: m for m in live if not m.absorbed}
        skip = set()
        for m in live:
            skip.update(m.ops)
        for g in self.moe:
            if g.disabled:
                continue
            self.roots[g.key] = g
            skip.update(g.skip_keys)
        self.skip = frozenset(skip)
        self.active = bool(self.roots)


def _hoist(v):
    """Follow a value out of the loops that merely carry it around: a while
    body argument whose carry is returned unchanged stands for the loop's
    initial operand (reference qmm.py:714-740)."""
    for _ in range(8):
        if not v.is_block_arg:
            return v
        op = v.block.parent_op
        if op is None or op.name != "stablehlo.while":
            return v
        body = op.regions[1]
        if v.block is not body and v.block is not op.regions[0]:
            return v
        if body.terminator.operands[v.index] is not body.args[v.index]:
            return v
        v = op.operands[v.index]
    return v


def _closure(values, main_args, ops, arg_indices, register=()):
    """Backward closure of `values` down to @main's arguments and constants
    (reference qmm.py:743-777)."""
    for o in register:
        ops[_key(o)] = o
    stack = list(values)
    seen = set()
    while stack:
        v = stack.pop()
        if v in seen:
            continue
        seen.add(v)
        if v.is_block_arg:
            idx = main_args.get(v)
            if idx is not None:
                arg_indices.add(idx)
                continue
            outer = _hoist(v)
            if outer is v:
                raise _Reject("operand depends on an inner block argument")
            stack.append(outer)
            continue
        o = v.op
        if o.name in _OPAQUE:
            raise _Reject(f"operand subtree contains {o.name}")
        ops.setdefault(_key(o), o)
        stack.extend(o.operands)


def _finish(ctx, m, root, absorb, dot, qside=1, required=(), register=()):
    """Fill in `m` for a dot whose operand `qside` is the quantized one
    (reference qmm.py:780-841)."""
    lb, rb, lc, rc = ir.dot_dims(dot)
    (qb, qc), (ab, ac) = (((rb, rc), (lb, lc)) if qside == 1 else ((lb, lc), (rb, rc)))
    if (qb or ab) and not _BATCH:
        raise _Reject("batching dimensions")
    quant, act = dot.operands[qside], dot.operands[1 - qside]
    if _el(act) not in FLOAT_ELS or _el(act) == "f64":
        raise _Reject(f"activation element type {_el(act)}")
    out_el = _el(root.results[0])
    if out_el not in FLOAT_ELS or out_el == "f64":
        raise _Reject(f"result element type {out_el}")
    qshape, ashape = _shape(quant), _shape(act)
    if [ashape[d] for d in ab] != [qshape[d] for d in qb]:
        raise _Reject("batching dimensions disagree")
    afree = [d for d in range(len(ashape)) if d not in ac and d not in ab]
    qfree = [d for d in range(len(qshape)) if d not in qc and d not in qb]
    B = _prod(ashape[d] for d in ab)
    M, K, N = (_prod(ashape[d] for d in afree), _prod(ashape[d] for d in ac),
               _prod(qshape[d] for d in qfree))
    if B == 0 or M == 0 or K == 0 or N == 0:
        raise _Reject("empty matmul")
    if K % _GROUP_SIZES[-1]:
        raise _Reject(f"K={K} is not a multiple of {_GROUP_SIZES[-1]}")
    if K != _prod(qshape[d] for d in qc):
        raise _Reject("contracting dimensions disagree")
    m.root = root
    m.key = _key(root)
    m.lhs = act
    m.swapped = qside == 0
    m.lperm = ab + afree + ac
    m.rperm = qb + qfree + qc
    m.rshape = qshape
    m.bshape = [ashape[d] for d in ab]
    m.mshape = [ashape[d] for d in afree]
    m.nshape = [qshape[d] for d in qfree]
    m.B, m.M, m.K, m.N = B, M, K, N
    m.out_dtype = out_el
    m.act_dtype = _el(act)
    m.name = (f"{M}x{K}x{N}" if not m.bshape
              else f"{'x'.join(map(str, m.bshape))}|{M}x{K}x{N}")
    if m.swapped:
        m.name += "'"
    main_args, donated = ctx
    arg_indices = set()
    _closure(absorb, main_args, m.ops, arg_indices, register)
    if arg_indices & donated:
        raise _Reject("quantized operand is donated (buffer may be reused)")
    m.arg_indices = tuple(sorted(arg_indices))
    m.required = [_key(o) for o in required] + [_key(o) for o in m.post]
    return m


def _has_int_leaf(v, limit=64):
    stack, seen = [v], set()
    while stack and len(seen) < limit:
        cur = stack.pop()
        if cur in seen:
            continue
        seen.add(cur)
        if _is_int(cur):
            return True
        o = cur.op
        if o is None or o.name in _OPAQUE:
            continue
        stack.extend(o.operands)
    return False


def _split_scaled(mul):
    """(values, scale) of `values * broadcast(one scale per 32 values)`
    (reference qmm.py:868-899)."""
    cands = []
    total = _prod(_shape(mul.results[0]))
    for i in (0, 1):
        v = mul.operands[i]
        if _el(v) not in FLOAT_ELS:
            raise _Reject(f"multiply operand element type {_el(v)}")
        base, dims = _bcast_chain(v)
        if dims is None:
            continue
        n = _prod(_shape(base))
        if n and n * _MXFP4_GROUP == total:
            cands.append((n, i))
    if not cands:
        raise _Reject(f"neither multiply operand broadcasts one scale per {_MXFP4_GROUP} values")
    if len(cands) == 2:
        raise _Reject("cannot tell the scale operand from the values")
    return mul.operands[1 - cands[0][1]], mul.operands[cands[0][1]]


def _try_affine(ctx, dot):
    reject = None
    for qside in (1, 0):
        try:
            return _try_affine_side(ctx, dot, qside)
        except _Reject as e:
            reject = reject or e
    raise reject


def _try_affine_side(ctx, dot, qside):
    qop = dot.operands[qside]
    base, post = _strip_shape(qop)
    mul = base.op
    if mul is None or mul.name != "stablehlo.multiply":
        raise _Reject("the operand is not a multiply")
    parsed = scale = None
    for i in (0, 1):
        parsed = _parse_codes(mul.operands[i])
        if parsed is not None:
            scale = mul.operands[1 - i]
            break
    m = Match()
    if parsed is None:
        values, scale = _split_scaled(mul)
        if not _has_int_leaf(values):
            raise _Reject("the scaled operand holds no integer codes")
        m.mode = "mxfp4"
        m.codes = values
    else:
        m.codes, m.zero, m.sub_range = parsed
    if _el(scale) not in FLOAT_ELS:
        raise _Reject(f"scale element type {_el(scale)}")
    m.scale = scale
    m.post = [o for o in post if o.name in _SHAPE_OPS]
    _finish(ctx, m, dot, [qop], dot, qside=qside, required=(mul,))
    return m


def _try_perchannel(ctx, div):
    num, den = div.operands
    dot = num.op
    if dot is None or dot.name != "stablehlo.dot_general":
        raise _Reject("divide numerator is not a dot")
    codes, post = _strip_shape(dot.operands[1])
    if not _is_int(codes):
        raise _Reject("dot rhs is not an integer code tensor")
    scale, dims = _bcast_chain(den)
    if dims is None:
        raise _Reject("divisor is not a broadcast")
    if _el(scale) not in FLOAT_ELS:
        raise _Reject("divisor is not float")
    lb, rb, lc, _rc = ir.dot_dims(dot)
    if lb or rb:
        raise _Reject("batching dimensions")
    nm = len(_shape(dot.operands[0])) - len(lc)
    if any(d < nm for d in dims):
        raise _Reject("divisor depends on the batch axis")
    m = Match()
    m.recip = True
    m.codes = codes
    m.scale = scale
    m.bcast_dims = [d - nm for d in dims]
    m.post = [o for o in post if o.name in _SHAPE_OPS]
    _finish(ctx, m, div, [dot.operands[1], den], dot, required=(dot,), register=(dot,))
    return m


def _prune(cands):
    """Which absorbed ops may really be skipped: an op only if every consumer
    is skipped too or is a rewritten root; a candidate whose required ops
    cannot be skipped is dropped (reference qmm.py:991-1039)."""
    live = list(cands)
    while True:
        ops = {}
        for m in live:
            ops.update(m.ops)
        roots = {m.key for m in live}
        work = deque(ops)
        while work:
            key = work.popleft()
            op = ops.get(key)
            if op is None:
                continue
            keep = True
            for r in op.results:
                for u in r.uses:
                    ukey = _key(u)
                    if ukey is None or (ukey not in ops and ukey not in roots):
                        keep = False
                        break
                if not keep:
                    break
            if keep:
                continue
            del ops[key]
            for opd in op.operands:
                if opd.op is not None and _key(opd.op) in ops:
                    work.append(_key(opd.op))
        kept = []
        for m in live:
            if any(k not in ops for k in m.required):
                _debug(f"dropped {m.name} (reconstruction is used elsewhere)")
                continue
            kept.append(m)
        if len(kept) == len(live):
            for m in live:
                m.ops = {k: v for k, v in m.ops.items() if k in ops}
            return live
        live = kept


def analyze(interp) -> State:
    """Structural analysis of a program, once.  Never touches values
    (reference qmm.py:1042-1091)."""
    st = interp._qmm
    if st is not None:
        return st
    st = State()
    interp._qmm = st
    try:
        if not QMM_ENABLED:
            raise _Reject("METALJAX_QMM=0")
        main = interp._main_block()
        ctx = ({a: i for i, a in enumerate(main.args)}, set(interp.donated_args))
        cands = []
        for block in ir.walk_blocks(main):
            for o in block.ops:
                try:
                    if o.name == "stablehlo.dot_general":
                        cands.append(_try_affine(ctx, o))
                    elif o.name == "stablehlo.divide":
                        cands.append(_try_perchannel(ctx, o))
                except _Reject:
                    pass
        absorbed = set()
        for m in cands:
            absorbed.update(m.ops)
        cands = [m for m in cands if m.key not in absorbed]
        st.matches = _prune(cands) if cands else []
        STATS["recognized"] += len(st.matches)
        if st.matches:
            _debug(f"{len(st.matches)} quantized matmul(s) recognized")
    except _Reject:
        st.matches = []
    except Exception as e:          # analysis must never break a program
        _debug(f"analysis failed ({e})")
        st.matches = []
    st.rebuild()
    interp.invalidate_plans()
    return st


# --------------------------------------------------------------------------
# first-execute verification + packing (host side, numpy)
# --------------------------------------------------------------------------

def _eval(interp, value, env):
    """Evaluate an operand subtree on concrete arguments with the
    interpreter's own handlers (reference qmm.py:1130-1176)."""
    if value in env:
        return env[value]
    if value.is_block_arg:
        outer = _hoist(value)
        if outer is value:
            raise _Reject("unbound value in operand subtree")
        env[value] = _eval(interp, outer, env)
        return env[value]
    # iterative post-order walk (reconstruction chains can be deep)
    stack = [value]
    while stack:
        v = stack[-1]
        if v in env:
            stack.pop()
            continue
        if v.is_block_arg:
            outer = _hoist(v)
            if outer is v:
                raise _Reject("unbound value in operand subtree")
            if outer in env:
                env[v] = env[outer]
                stack.pop()
            else:
                stack.append(outer)
            continue
        o = v.op
        missing = [x for x in o.operands if x not in env]
        if missing:
            stack.extend(missing)
            continue
        handler = REGISTRY.get(o.name)
        if handler is None or o.name in _OPAQUE:
            raise _Reject(f"no handler for {o.name}")
        out = handler(interp, o, [env[x] for x in o.operands], env)
        if not isinstance(out, (list, tuple)):
            out = [out]
        for r, val in zip(o.results, out):
            env[r] = val
        stack.pop()
    return env[value]


def _replay(a: np.ndarray, post):
    for o in post:
        if o.name == "stablehlo.reshape":
            a = a.reshape(o.results[0].type.shape)
        else:
            a = np.transpose(a, ir.i64_list(o, "permutation"))
    return a


def _to_nk(x: HostArray, m) -> np.ndarray:
    """A rhs-shaped tensor as the [(B,) N, K] matrix the kernels want
    (reference qmm.py:1188-1201)."""
    a = _replay(x.a, m.post)
    if list(a.shape) != m.rshape:
        raise _Reject(f"expected rhs shape {m.rshape}, got {list(a.shape)}")
    shape = (m.bshape + [m.N, m.K]) if m.bshape else [m.N, m.K]
    return np.ascontiguousarray(np.transpose(a, m.rperm).reshape(shape))


def _typed(a: np.ndarray, el: str):
    """Host values in the representation the pack primitives take."""
    if el == "bf16":
        return BF16Array.from_f32(a)
    if el == "f16":
        return np.ascontiguousarray(a, np.float16)
    return np.ascontiguousarray(a)


def _device(a):
    """Packed arrays live on the GPU when there is one (they are inputs of the
    fused kernel); on a machine without one they stay host arrays, which is
    enough for everything but `emit`."""
    import torch
    if not torch.cuda.is_available():
        return a
    if isinstance(a, BF16Array):
        return torch.from_numpy(a.bits.view(np.int16).copy()).cuda().view(torch.bfloat16)
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32).copy()).cuda()
    return torch.from_numpy(a.copy()).cuda()


def _build_mxfp4_pack(interp, m, env, leaves):
    """Verify and repack an MXFP4 weight (reference qmm.py:1723-1770)."""
    gs = _MXFP4_GROUP
    if m.K % gs:
        raise _Reject(f"K={m.K} is not a multiple of {gs}")
    sv = _eval(interp, m.scale, env)
    scale_map = _to_nk(sv, m)
    perm = None
    if not packing.group_const(scale_map, gs):
        perm = packing.regroup(m.K, (scale_map,))
        if perm is not None:
            scale_map = packing.take_k(scale_map, perm)
        if not packing.group_const(scale_map, gs):
            raise _Reject(f"MXFP4 scales are not constant within a group of {gs}")
    sbytes = packing.mxfp4_scale_bytes(packing.group_heads(scale_map, gs))
    vv = _eval(interp, m.codes, env)
    values = _typed(_to_nk(vv, m), vv.el)
    if perm is not None:
        values = packing.take_k(values, perm)
    w = packing.pack_codes(packing.mxfp4_codes(values), 4)
    return _finalize(leaves, w, sbytes, None, perm, gs, 4, "mxfp4")


def _build_affine_pack(interp, m, env, leaves):
    """Verify and repack a `scale * (code - zero)` weight
    (reference qmm.py:1773-1915)."""
    cv = _eval(interp, m.codes, env)
    codes = _to_nk(cv, m).astype(np.int64)
    lo, hi = int(codes.min()), int(codes.max())
    if hi - lo < 16:
        bits = 4
    elif hi - lo < 256:
        bits = 8
    else:
        raise _Reject(f"codes span [{lo}, {hi}]: more than 8 bits")
    offset = 1 << (bits - 1)
    if lo + offset < 0 or hi + offset >= (1 << bits):
        offset = -lo
    perm = None
    if m.recip:
        sv = _eval(interp, m.scale, env)
        scale_kind = sv.el if sv.el in ("bf16", "f16") else None
        s = sv.a.astype(np.float32)
        interim = [1] * len(m.nshape)
        dims = m.bcast_dims
        if dims != sorted(dims):
            s = np.transpose(s, sorted(range(len(dims)), key=lambda i: dims[i]))
            dims = sorted(dims)
        for i, d in enumerate(dims):
            interim[d] = s.shape[i]
        s = np.broadcast_to(s.reshape(interim), m.nshape).reshape(m.N, 1)
        scales = (np.float32(1.0) / s).astype(np.float32)
        gs = next((g for g in _GROUP_SIZES if m.K % g == 0), None)
        if gs is None:
            raise _Reject(f"K={m.K} has no legal group size")
        scales = np.ascontiguousarray(np.broadcast_to(scales, (m.N, m.K // gs)))
        zeros = None
    else:
        g0 = _GROUP_SIZES[-1]
        sv = _eval(interp, m.scale, env)
        scale_kind = sv.el if sv.el in ("bf16", "f16") else None
        scale_map = _to_nk(sv, m)
        zero_map = None
        if m.zero is not None:
            zero_map = _to_nk(_eval(interp, m.zero, env), m)
        if not packing.group_const(scale_map, g0) or (
                zero_map is not None and not packing.group_const(zero_map, g0)):
            perm = packing.regroup(m.K, (scale_map, zero_map))
            note = ""
            if perm is not None:
                scale_map = packing.take_k(scale_map, perm)
                if zero_map is not None:
                    zero_map = packing.take_k(zero_map, perm)
                note = " (even regrouped)"
            if not packing.group_const(scale_map, g0) or (
                    zero_map is not None and not packing.group_const(zero_map, g0)):
                raise _Reject(f"scales/zeros are not constant within any group{note}")
        scales = packing.group_heads(scale_map, g0)
        zeros = None if zero_map is None else packing.group_heads(zero_map, g0)
        gs = packing.pick_group_heads(m.K, scales, zeros)
        if gs is None:
            raise _Reject("scales/zeros are not constant within any group")
        if gs != g0:
            scales = packing.group_heads(scales, gs // g0)
            if zeros is not None:
                zeros = packing.group_heads(zeros, gs // g0)
        if zeros is not None:
            zeros = zeros.astype(np.float32)
            if not bool((zeros == np.round(zeros)).all()):
                raise _Reject("zero points are not integers")
            if bool((np.abs(zeros) > 32768).any()):
                raise _Reject("zero points out of range")
            if m.sub_range is not None:
                zlo, zhi = int(zeros.min()), int(zeros.max())
                if (lo - zhi) < m.sub_range[0] or (hi - zlo) > m.sub_range[1]:
                    raise _Reject("integer zero-point subtraction can wrap")
    if perm is not None:
        codes = packing.take_k(codes, perm)
    w = packing.pack_codes((codes + offset).astype(np.uint8), bits)
    scales, biases = packing.scale_bias(scales, zeros, offset, scale_kind)
    return _finalize(leaves, w, scales, biases, perm, gs, bits, "affine")


# content-addressed sharing of identical packs (tied / duplicated weights)
_SHARED = {}


def _digest(arrays):
    h = hashlib.blake2b(digest_size=16)
    for a in arrays:
        if a is None:
            h.update(b"-")
            continue
        b = np.ascontiguousarray(a.bits if isinstance(a, BF16Array) else a)
        h.update(str((isinstance(a, BF16Array), b.dtype.str, b.shape)).encode())
        h.update(b.tobytes())
    return h.hexdigest()


def _finalize(leaves, w, scales, biases, perm, gs, bits, mode):
    """Host-packed arrays -> a pack holding device arrays.  A pack whose bytes
    equal those of a live earlier pack (tied or duplicated weights) shares its
    arrays instead of uploading a copy (reference qmm.py:1656-1704)."""
    perm = None if perm is None else np.ascontiguousarray(perm, np.int32)
    key = (mode, gs, bits, _digest([w, scales, biases, perm])) if _SHARE else None
    old = None
    if key is not None:
        ref = _SHARED.get(key)
        old = ref() if ref is not None else None
    if old is not None:
        STATS["shared"] += 1
        pk = _Pack(leaves, old.w, old.scales, old.biases, old.perm, gs, bits, mode)
        pk._origin = old
        return pk
    pk = _Pack(leaves, _device(w), _device(scales), None if biases is None else _device(biases),
               None if perm is None else _device(perm), gs, bits, mode)
    if key is not None:
        _SHARED[key] = weakref.ref(pk)
    return pk


def _record_pack(m, pk):
    STATS["packs"] += 1
    if pk.perm is not None:
        STATS["perms"] += 1
    if pk.mode == "mxfp4":
        STATS["mxfp4"] += 1
    if m.bshape:
        STATS["batched"] += 1
    _debug(f"packed {m.name} mode={pk.mode} bits={pk.bits} group={pk.gs}"
           f"{' regrouped' if pk.perm is not None else ''}")
    return pk


def _check_kernel(m, pk):
    """Refuse at pack time what the kernels do not serve, so that the dot runs
    literally instead of failing at every step."""
    if m.act_dtype != "bf16":
        raise _Reject(f"activation dtype {m.act_dtype}: the kernels take bf16 activations")
    if m.out_dtype not in ("bf16", "f16", "f32"):
        raise _Reject(f"result dtype {m.out_dtype}")


def _build_pack(interp, m, args, leaves):
    env = dict(zip(interp._main_block().args, args))
    pk = (_build_mxfp4_pack(interp, m, env, leaves) if m.mode == "mxfp4"
          else _build_affine_pack(interp, m, env, leaves))
    _check_kernel(m, pk)
    return _record_pack(m, pk)


# ---- cross-executable build cache: (canonical text of the reconstruction
# subtree, identity of the buffers it reads) -> pack
_BUILT = {}


def _fingerprint(m):
    """Canonical serialization of the reconstruction subtree: ops in a
    deterministic post-order, operands by position, leaves by argument slot
    (reference qmm.py:2022-2268 keeps the same two-part key)."""
    if m.fp is not None:
        return m.fp
    ids, lines = {}, []
    arg_slot = {}

    def visit(v):
        v = _hoist(v) if v.is_block_arg else v
        if v in ids:
            return ids[v]
        if v.is_block_arg:
            slot = arg_slot.setdefault(v, len(arg_slot))
            ids[v] = f"a{slot}:{v.type}"
            return ids[v]
        o = v.op
        if o.name in _OPAQUE:
            raise _Reject("opaque op in subtree")
        opnds = [visit(x) for x in o.operands]
        attrs = sorted((k, repr(val)) for k, val in o.attrs.items())
        n = len(lines)
        lines.append(f"{n}={o.name}{attrs}({','.join(opnds)})->{[str(r.type) for r in o.results]}")
        for i, r in enumerate(o.results):
            ids[r] = f"%{n}.{i}"
        return ids[v]

    try:
        parts = [visit(x) for x in (m.codes, m.zero, m.scale) if x is not None]
        extra = (m.mode, m.recip, m.rperm, m.rshape, m.bcast_dims,
                 [(o.name, repr(sorted(o.attrs.items(), key=str))) for o in m.post])
        m.fp = ("\n".join(lines) + "|" + ",".join(parts) + "|" + repr(extra),
                [a.index for a in sorted(arg_slot, key=arg_slot.get)])
    except (_Reject, RecursionError):
        m.fp = False
        STATS["build_declines"] += 1
    return m.fp


def _build_key(m, args):
    if not _BUILD_CACHE:
        return None, None
    fp = _fingerprint(m)
    if not fp:
        return None, None
    text, slots = fp
    keyleaves = [args[i] for i in slots]
    return (text, tuple(id(a) for a in keyleaves)), keyleaves


def _cached_build(key, keyleaves):
    hit = _BUILT.get(key)
    if hit is None:
        return None
    refs, pref = hit
    pk = pref()
    if pk is None or len(refs) != len(keyleaves) or not all(r() is a for r, a in zip(refs, keyleaves)):
        _BUILT.pop(key, None)
        return None
    return pk


def _remember_build(key, keyleaves, pk):
    _BUILT[key] = ([weakref.ref(a) for a in keyleaves], weakref.ref(pk))


def _resolve(interp, m, args):
    """(pack, freshly_built) for these argument buffers
    (reference qmm.py:2271-2302)."""
    leaves = [args[i] for i in m.arg_indices]
    for i, pk in enumerate(m.packs):
        if pk.matches(leaves):
            if i:
                m.packs.insert(0, m.packs.pop(i))
            return pk, False
    key, keyleaves = _build_key(m, args)
    if key is not None:
        old = _cached_build(key, keyleaves)
        if old is not None:
            STATS["build_hits"] += 1
            pk = _Pack(leaves, old.w, old.scales, old.biases, old.perm, old.gs, old.bits, old.mode)
            pk._origin = old                       # keeps the shared build alive
            m.packs.insert(0, pk)
            del m.packs[_MAX_PACKS:]
            return pk, False
    m.repacks += 1
    if m.repacks > _MAX_REPACKS:
        raise _Reject(f"operands changed {m.repacks} times; repacking costs more than the "
                      "chain it replaces")
    pk = _build_pack(interp, m, args, leaves)
    if key is not None:
        _remember_build(key, keyleaves, pk)
    m.packs.insert(0, pk)
    del m.packs[_MAX_PACKS:]
    return pk, True


def prologue(interp, args) -> bool:
    """Pack every recognized weight against these arguments, eagerly.  Returns
    True when the set of rewritten dots changed (reference qmm.py:2305-2387)."""
    st = interp._qmm
    if st is None:
        st = analyze(interp)
    if not st.matches and not st.moe:
        return False
    changed = False
    values = []
    for m in st.matches:
        if m.disabled:
            continue
        try:
            pk, _fresh = _resolve(interp, m, args)
        except Exception as e:
            from ._lib import QmmLibraryError
            if isinstance(e, QmmLibraryError):
                raise
            m.disabled = True
            changed = True
            STATS["fallbacks"] += 1
            _debug(f"{m.name} falls back to the literal chain ({e})")
            continue
        if (m.mode, m.gs, m.bits, m.has_perm) != (pk.mode, pk.gs, pk.bits, pk.perm is not None):
            changed = changed or m.gs != 0
            m.mode, m.gs, m.bits = pk.mode, pk.gs, pk.bits
            m.has_perm = pk.perm is not None
        m.slot = len(values)
        arrays = pk.arrays()
        m.nvals = len(arrays)
        values.extend(arrays)
    if changed:
        st.rebuild()
        interp.invalidate_plans()
    st.values = values
    return changed


# --------------------------------------------------------------------------
# runtime
# --------------------------------------------------------------------------

def values(interp):
    st = getattr(interp, "_qmm", None)
    return st.values if st is not None else ()


def push(interp, vals):
    st = getattr(interp, "_qmm", None)
    if st is None or not st.values:
        return None
    prev = st.values
    st.values = list(vals)
    return (prev,)


def pop(interp, token):
    if token is not None:
        interp._qmm.values = token[0]


def pack_arrays(interp, m):
    st = interp._qmm
    return st.values[m.slot:m.slot + m.nvals]


def emit_reads(m):
    """The env values `emit` reads: exactly the activation operand
    (reference qmm.py:2424-2442)."""
    if not isinstance(m, Match):
        from . import moe
        return moe.emit_reads(m)
    return (m.lhs,)


def emit_bytes(m) -> int:
    """Device bytes `emit` materializes beyond the root's own result: one copy
    of the activation (reference qmm.py:2445-2466)."""
    if not isinstance(m, Match):
        from . import moe
        return moe.emit_bytes(m)
    return m.lhs.type.size * ir._EL_BYTES[m.lhs.type.el]


_TORCH_EL = None


def _torch_dtype(el):
    import torch
    return {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[el]


def to_device(v):
    """A runtime value as a device tensor (bf16 HostArrays become bfloat16)."""
    import torch
    if isinstance(v, torch.Tensor):
        return v if v.is_cuda else v.cuda()
    h = host(v)
    if h.el == "bf16":
        bits = packing.f32_to_bf16_bits(h.a).view(np.int16)
        return torch.from_numpy(np.ascontiguousarray(bits)).cuda().view(torch.bfloat16)
    return torch.from_numpy(np.ascontiguousarray(h.a)).cuda()


def emit(interp, m, env):
    """One fused quantized matmul in place of the whole dequant-and-dot
    (reference qmm.py:2469-2501)."""
    if not isinstance(m, Match):
        from . import moe
        return moe.emit(interp, m, env)
    from . import kernels
    st = interp._qmm
    vals = st.values[m.slot:m.slot + m.nvals]
    w, scales = vals[0], vals[1]
    biases = vals[2] if m.mode == "affine" else None
    x = to_device(env[m.lhs])
    if m.lperm != list(range(x.dim())):
        x = x.permute(m.lperm)
    x = x.reshape([m.B, m.M, m.K] if m.bshape else [m.M, m.K]).contiguous()
    if m.has_perm:
        x = kernels.take_k(x, vals[-1])
    y = kernels.quantized_matmul(x, w, scales, biases, transpose=True, group_size=m.gs,
                                 bits=m.bits, mode=m.mode, out_dtype=_torch_dtype(m.out_dtype))
    if m.swapped:
        y = y.transpose(-1, -2).reshape(m.bshape + m.nshape + m.mshape)
    else:
        y = y.reshape(m.bshape + m.mshape + m.nshape)
    return [y]
