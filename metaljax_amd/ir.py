"""A small StableHLO-text front end: module text -> an SSA graph.

The quantized-matmul recognizer only needs to walk operands, users, regions
and a handful of attributes, so this is a plain-Python graph with identity
hashing, not an MLIR binding.  It reads the textual forms jax prints for the
ops that appear between integer weight codes and a dot (pretty forms, plus the
generic quoted form for gather / while and anything else), see the `_PRETTY`
table.  The reference walks the same structure through jaxlib's MLIR objects
(reference src/metaljax/qmm.py:472-485, src/metaljax/_ir.py:15-159).
"""

from __future__ import annotations

import re
from dataclasses import dataclass, field

import numpy as np


class ParseError(ValueError):
    pass


# ------------------------------------------------------------------ types ----

@dataclass(frozen=True)
class TensorType:
    shape: tuple
    el: str

    def __str__(self):
        return "tensor<" + "x".join([*map(str, self.shape), self.el]) + ">"

    @property
    def size(self) -> int:
        n = 1
        for d in self.shape:
            n *= d
        return n


_EL_BYTES = {"i1": 1, "i4": 1, "ui4": 1, "i8": 1, "ui8": 1, "i16": 2, "ui16": 2, "i32": 4,
             "ui32": 4, "i64": 8, "ui64": 8, "f16": 2, "bf16": 2, "f32": 4, "f64": 8}


def parse_type(text: str) -> TensorType:
    text = text.strip()
    m = re.fullmatch(r"tensor<(.*)>", text, re.S)
    if not m:
        if text in _EL_BYTES:           # a bare element type (scalar attributes)
            return TensorType((), text)
        raise ParseError(f"unsupported type {text!r}")
    body = m.group(1).split(",")[0].strip()      # drop encodings
    parts = body.split("x")
    el = parts[-1]
    if el not in _EL_BYTES:
        raise ParseError(f"unsupported element type {el!r} in {text!r}")
    try:
        shape = tuple(int(p) for p in parts[:-1])
    except ValueError as e:
        raise ParseError(f"dynamic shape in {text!r}") from e
    return TensorType(shape, el)


# ------------------------------------------------------------------ graph ----

class Value:
    """An SSA value: an op result or a block argument.  Hashes by identity."""

    __slots__ = ("type", "op", "index", "block", "uses", "name")

    def __init__(self, type_, op=None, index=0, block=None, name=""):
        self.type = type_
        self.op = op              # defining op (None for block arguments)
        self.index = index        # result number / argument number
        self.block = block        # owning block, for block arguments
        self.uses = []            # ops that read this value (one entry per operand slot)
        self.name = name

    @property
    def is_block_arg(self) -> bool:
        return self.op is None

    def __repr__(self):
        return f"%{self.name}:{self.type}"


class Op:
    __slots__ = ("name", "operands", "results", "attrs", "regions", "block", "pos")

    def __init__(self, name, operands, result_types, attrs, regions, names=()):
        self.name = name
        self.operands = list(operands)
        self.results = [Value(t, self, i, name=(names[i] if i < len(names) else ""))
                        for i, t in enumerate(result_types)]
        self.attrs = attrs
        self.regions = regions    # list of Block
        self.block = None
        self.pos = -1
        for v in self.operands:
            v.uses.append(self)
        for r in regions:
            r.parent_op = self

    def __repr__(self):
        return f"<{self.name} -> {[str(r.type) for r in self.results]}>"


class Block:
    __slots__ = ("args", "ops", "parent_op")

    def __init__(self, args=()):
        self.args = list(args)
        self.ops = []
        self.parent_op = None
        for i, a in enumerate(self.args):
            a.block, a.index = self, i

    def append(self, op):
        op.block, op.pos = self, len(self.ops)
        self.ops.append(op)

    @property
    def terminator(self):
        return self.ops[-1]


@dataclass
class Func:
    name: str
    body: Block
    result_types: list
    arg_attrs: list
    visibility: str = "public"


@dataclass
class Module:
    funcs: dict = field(default_factory=dict)
    text: str = ""

    @property
    def main(self) -> Func:
        if "main" in self.funcs:
            return self.funcs["main"]
        pub = [f for f in self.funcs.values() if f.visibility != "private"]
        if len(pub) == 1:
            return pub[0]
        raise ParseError("no @main function")


# -------------------------------------------------------------- tokenizer ----

_TOKEN = re.compile(r"""
    (?P<ws>\s+|//[^\n]*)
  | (?P<arrow>->)
  | (?P<ssa>%[A-Za-z0-9_.$-]+(?:\#\d+)?)
  | (?P<sym>@[A-Za-z0-9_.$-]+|@"[^"]*")
  | (?P<caret>\^[A-Za-z0-9_.$-]+)
  | (?P<str>"(?:[^"\\]|\\.)*")
  | (?P<num>[-+]?(?:0x[0-9A-Fa-f]+|(?:\d+\.\d*|\.\d+|\d+)(?:[eE][-+]?\d+)?))
  | (?P<hash>\#[A-Za-z0-9_.]+)
  | (?P<id>[A-Za-z_][A-Za-z0-9_.$]*)
  | (?P<punct>[(){}\[\]<>,:=*?!|+-])
""", re.X)

_BALANCED_HEADS = {"tensor", "dense", "array", "loc", "complex", "tuple"}


def _tokenize(text):
    toks = []
    i, n = 0, len(text)
    while i < n:
        m = _TOKEN.match(text, i)
        if not m:
            raise ParseError(f"cannot tokenize at {text[i:i + 40]!r}")
        kind = m.lastgroup
        val = m.group(kind)
        i = m.end()
        if kind == "ws":
            continue
        if kind in ("id", "hash") and i < n and text[i] in "<(" and (
                kind == "hash" or val in _BALANCED_HEADS):
            if text[i] == "(" and val != "loc":
                toks.append((kind, val))
                continue
            # swallow the balanced <...> / (...) payload into one token
            open_, close_ = text[i], ">" if text[i] == "<" else ")"
            depth, j = 0, i
            while j < n:
                c = text[j]
                if c == '"':
                    j = text.index('"', j + 1)
                elif c == "-" and text[j:j + 2] == "->":
                    j += 1
                elif c == open_:
                    depth += 1
                elif c == close_:
                    depth -= 1
                    if depth == 0:
                        break
                j += 1
            payload = text[i + 1:j]
            i = j + 1
            if val == "loc":
                continue
            toks.append(("balanced", (val, payload)))
            continue
        toks.append((kind, val))
    toks.append(("eof", None))
    return toks


# ----------------------------------------------------------------- parser ----

_SAME_TYPE_BINARY = {
    "add", "subtract", "multiply", "divide", "and", "or", "xor", "shift_left",
    "shift_right_logical", "shift_right_arithmetic", "maximum", "minimum", "power", "remainder",
    "atan2"}
_UNARY = {
    "negate", "abs", "exponential", "log", "sqrt", "rsqrt", "tanh", "logistic", "floor", "ceil",
    "not", "sign", "round_nearest_even", "round_nearest_afz", "cosine", "sine", "log_plus_one",
    "exponential_minus_one", "is_finite", "popcnt", "count_leading_zeros", "cbrt", "tan"}


class _Parser:
    def __init__(self, text):
        self.toks = _tokenize(text)
        self.i = 0
        self.module = Module(text=text)
        self.scopes = []          # list of {ssa name: Value | [Value]}

    # -- token helpers
    def peek(self, k=0):
        return self.toks[self.i + k]

    def next(self):
        t = self.toks[self.i]
        self.i += 1
        return t

    def accept(self, kind, val=None):
        t = self.toks[self.i]
        if t[0] == kind and (val is None or t[1] == val):
            self.i += 1
            return t
        return None

    def expect(self, kind, val=None):
        t = self.accept(kind, val)
        if t is None:
            got = self.toks[self.i]
            raise ParseError(f"expected {val or kind}, got {got[1]!r} (token {self.i})")
        return t

    # -- scopes
    def define(self, name, value):
        self.scopes[-1][name] = value

    def lookup(self, ref):
        name, _, idx = ref[1:].partition("#")
        for sc in reversed(self.scopes):
            if name in sc:
                v = sc[name]
                if isinstance(v, list):
                    return v[int(idx)] if idx else v[0]
                return v
        raise ParseError(f"use of undefined value %{name}")

    # -- pieces
    def type_(self):
        t = self.next()
        if t[0] == "balanced" and t[1][0] == "tensor":
            return parse_type(f"tensor<{t[1][1]}>")
        if t[0] == "id" and t[1] in _EL_BYTES:
            return TensorType((), t[1])
        raise ParseError(f"expected a tensor type, got {t[1]!r}")

    def type_list(self):
        """`T` | `(T, T, ...)` (each optionally followed by an attribute dict)."""
        out = []
        if self.accept("punct", "("):
            while not self.accept("punct", ")"):
                out.append(self.type_())
                if self.peek() == ("punct", "{"):
                    self.attr_dict()
                self.accept("punct", ",")
        else:
            out.append(self.type_())
        return out

    def int_list(self):
        self.expect("punct", "[")
        out = []
        while not self.accept("punct", "]"):
            out.append(int(self.expect("num")[1], 0))
            self.accept("punct", ",")
        return out

    def attr_value(self, typed=True):
        t = self.peek()
        if t == ("punct", "["):
            self.next()
            out = []
            while not self.accept("punct", "]"):
                out.append(self.attr_value())
                self.accept("punct", ",")
            return out
        if t == ("punct", "{"):
            return self.attr_dict()
        self.next()
        if t[0] == "num":
            v = float(t[1]) if re.search(r"[.eE]", t[1]) and not t[1].lower().startswith("0x") else int(t[1], 0)
            if typed and self.accept("punct", ":"):
                self.type_()
            return v
        if t[0] == "str":
            return t[1][1:-1]
        if t[0] == "sym":
            return t[1]
        if t[0] == "id":
            if t[1] in ("true", "false"):
                return t[1] == "true"
            if t[1] == "unit":
                return True
            return t[1]
        if t[0] == "balanced":
            head, payload = t[1]
            if head == "array":
                body = payload.split(":", 1)[1] if ":" in payload else ""
                return [int(x, 0) for x in body.replace(",", " ").split()]
            if head == "dense":
                ty = None
                if typed and self.accept("punct", ":"):
                    ty = self.type_()
                return ("dense", payload, ty)
            if head.startswith("#"):
                return (head, _hash_fields(payload))
            return (head, payload)
        if t[0] == "hash":
            return t[1]
        raise ParseError(f"unsupported attribute value {t[1]!r}")

    def attr_dict(self):
        self.expect("punct", "{")
        out = {}
        while not self.accept("punct", "}"):
            k = self.next()
            if k[0] not in ("id", "str"):
                raise ParseError(f"bad attribute key {k[1]!r}")
            key = k[1].strip('"')
            out[key] = self.attr_value() if self.accept("punct", "=") else True
            self.accept("punct", ",")
        return out

    def operand_list(self, close=None):
        out = []
        while self.peek()[0] == "ssa":
            out.append(self.lookup(self.next()[1]))
            if not self.accept("punct", ","):
                break
        return out

    # -- module / functions
    def parse(self):
        while self.peek()[0] != "eof" and self.peek() not in (("id", "module"), ("id", "func.func")):
            self.next()                         # location aliases ahead of the module
        if self.accept("id", "module"):
            self.accept("sym")
            if self.accept("id", "attributes"):
                self.attr_dict()
            self.expect("punct", "{")
            while not self.accept("punct", "}"):
                if self.peek() != ("id", "func.func"):
                    self.skip_statement()       # sdy.mesh and other module-level metadata
                    continue
                self.func()
        else:
            while self.peek() == ("id", "func.func"):
                self.func()
        return self.module

    def skip_statement(self):
        """Skip a module-level statement this front end has no use for."""
        self.next()
        depth = 0
        while True:
            t = self.peek()
            if t[0] == "eof":
                return
            if depth == 0 and (t == ("id", "func.func") or t == ("punct", "}")):
                return
            if t[0] == "punct" and t[1] in "({[<":
                depth += 1
            elif t[0] == "punct" and t[1] in ")}]>":
                depth -= 1
            self.next()

    def func(self):
        self.expect("id", "func.func")
        vis = "public"
        if self.peek()[0] == "id" and self.peek()[1] in ("public", "private", "nested"):
            vis = self.next()[1]
        name = self.expect("sym")[1][1:]
        self.expect("punct", "(")
        args, arg_attrs, names = [], [], []
        while not self.accept("punct", ")"):
            ref = self.expect("ssa")[1]
            self.expect("punct", ":")
            ty = self.type_()
            attrs = self.attr_dict() if self.peek() == ("punct", "{") else {}
            args.append(Value(ty, name=ref[1:]))
            names.append(ref[1:])
            arg_attrs.append(attrs)
            self.accept("punct", ",")
        results = self.type_list() if self.accept("arrow") else []
        if self.accept("id", "attributes"):
            self.attr_dict()
        body = Block(args)
        self.scopes.append({n: a for n, a in zip(names, args)})
        self.expect("punct", "{")
        self.block_ops(body)
        self.scopes.pop()
        self.module.funcs[name] = Func(name, body, results, arg_attrs, vis)

    def block_ops(self, block):
        """Ops up to (and consuming) the closing brace."""
        while not self.accept("punct", "}"):
            block.append(self.op())

    def region_block(self, pre_args=None):
        """`{ [^bb(%a: T, ...):] ops }`; `pre_args` are (name, Value) already bound."""
        self.expect("punct", "{")
        args, names = [], []
        if pre_args:
            names, args = [n for n, _ in pre_args], [v for _, v in pre_args]
        if self.peek()[0] == "caret":
            self.next()
            if self.accept("punct", "("):
                while not self.accept("punct", ")"):
                    ref = self.expect("ssa")[1]
                    self.expect("punct", ":")
                    args.append(Value(self.type_(), name=ref[1:]))
                    names.append(ref[1:])
                    self.accept("punct", ",")
            self.expect("punct", ":")
        blk = Block(args)
        self.scopes.append({n: a for n, a in zip(names, args)})
        self.block_ops(blk)
        self.scopes.pop()
        return blk

    # -- operations
    def op(self):
        res_names, counts = [], []
        while self.peek()[0] == "ssa" and self.peek(1) in (("punct", ","), ("punct", "="), ("punct", ":")):
            ref = self.next()[1][1:]
            n = 1
            if self.accept("punct", ":"):
                n = int(self.expect("num")[1])
            res_names.append(ref)
            counts.append(n)
            if self.accept("punct", "="):
                break
            self.expect("punct", ",")
        t = self.next()
        if t[0] == "str":
            op = self.generic_op(t[1][1:-1])
        elif t[0] == "id":
            op = self.pretty_op(t[1])
        else:
            raise ParseError(f"expected an operation, got {t[1]!r}")
        # bind result names
        k = 0
        for ref, n in zip(res_names, counts):
            vals = op.results[k:k + n]
            if len(vals) != n:
                raise ParseError(f"{op.name}: {len(op.results)} results, names want more")
            for j, v in enumerate(vals):
                v.name = ref if n == 1 else f"{ref}#{j}"
            self.define(ref, vals[0] if n == 1 else vals)
            k += n
        return op

    def fn_type(self):
        """`: (T, ...) -> T | (T, ...)`; returns (ins, outs)."""
        self.expect("punct", ":")
        ins = self.type_list()
        self.expect("arrow")
        return ins, self.type_list()

    def generic_op(self, name):
        self.expect("punct", "(")
        operands = self.operand_list()
        self.expect("punct", ")")
        attrs = {}
        if self.peek() == ("punct", "<") and self.peek(1) == ("punct", "{"):
            self.next()
            attrs.update(self.attr_dict())
            self.expect("punct", ">")
        regions = []
        if self.peek() == ("punct", "(") and self.peek(1) == ("punct", "{"):
            self.next()
            while True:
                regions.append(self.region_block())
                if not self.accept("punct", ","):
                    break
            self.expect("punct", ")")
        if self.peek() == ("punct", "{"):
            attrs.update(self.attr_dict())
        _, outs = self.fn_type()
        return Op(name, operands, outs, attrs, regions)

    def pretty_op(self, name):
        short = name.split(".", 1)[1] if "." in name else name
        if name in ("return", "func.return", "stablehlo.return"):
            operands = self.operand_list()
            if self.accept("punct", ":"):
                self.type_()
                while self.accept("punct", ","):
                    self.type_()
            return Op("return", operands, [], {}, [])
        if name in ("call", "func.call"):
            callee = self.expect("sym")[1][1:]
            self.expect("punct", "(")
            operands = self.operand_list()
            self.expect("punct", ")")
            _, outs = self.fn_type()
            return Op("func.call", operands, outs, {"callee": callee}, [])
        if name == "chlo.top_k":
            # `chlo.top_k(%x, k = 2) : tensor<..> -> (tensor<..>, tensor<..>)`
            self.expect("punct", "(")
            operands = [self.lookup(self.expect("ssa")[1])]
            self.expect("punct", ",")
            self.expect("id", "k")
            self.expect("punct", "=")
            k = int(self.expect("num")[1])
            self.expect("punct", ")")
            self.expect("punct", ":")
            self.type_()
            self.expect("arrow")
            return Op(name, operands, self.type_list(), {"k": k}, [])
        if not name.startswith("stablehlo."):
            return self.opaque_op(name)
        if short == "constant":
            val = self.attr_value()
            if not (isinstance(val, tuple) and val[0] == "dense"):
                raise ParseError("constant without a dense attribute")
            ty = val[2]
            return Op(name, [], [ty], {"value": val}, [])
        if short == "iota":
            self.expect("id", "dim")
            self.expect("punct", "=")
            d = int(self.expect("num")[1])
            self.expect("punct", ":")
            return Op(name, [], [self.type_()], {"iota_dimension": d}, [])
        if short == "while":
            return self.while_op()
        if short == "reduce":
            return self.reduce_op()
        if short == "compare":
            direction = self.expect("id")[1]
            self.expect("punct", ",")
            operands = self.operand_list()
            attrs = {"comparison_direction": direction}
            if self.peek()[0] == "id":
                attrs["compare_type"] = self.next()[1]
            _, outs = self.fn_type()
            return Op(name, operands, outs, attrs, [])
        if short == "composite":
            cname = self.expect("str")[1][1:-1]
            operands = self.operand_list()
            attrs = self.attr_dict() if self.peek() == ("punct", "{") else {}
            attrs["name"] = cname
            _, outs = self.fn_type()
            return Op(name, operands, outs, attrs, [])
        operands = self.operand_list()
        attrs = {}
        if short == "slice":
            self.expect("punct", "[")
            starts, limits, strides = [], [], []
            while not self.accept("punct", "]"):
                starts.append(int(self.expect("num")[1]))
                self.expect("punct", ":")
                limits.append(int(self.expect("num")[1]))
                strides.append(int(self.expect("num")[1]) if self.accept("punct", ":") else 1)
                self.accept("punct", ",")
            attrs = {"start_indices": starts, "limit_indices": limits, "strides": strides}
        # `, key = value` trailers (dims = [...], dim = n, sizes = [...], contracting_dims = ...)
        while self.peek()[0] == "id" and self.peek(1) == ("punct", "="):
            key = self.next()[1]
            self.next()
            if key in ("batching_dims", "contracting_dims"):
                a = self.int_list()
                self.expect("id", "x")
                attrs[key] = (a, self.int_list())
            elif self.peek() == ("punct", "["):
                vals = []
                self.next()
                while not self.accept("punct", "]"):
                    v = self.next()
                    vals.append(int(v[1], 0) if v[0] == "num" else v[1])
                    self.accept("punct", ",")
                attrs[key] = vals
            else:
                attrs[key] = self.attr_value(typed=False)
            self.accept("punct", ",")
        if self.peek() == ("punct", "{"):
            attrs.update(self.attr_dict())
        self.expect("punct", ":")
        if self.peek() == ("punct", "("):
            self.type_list()
            self.expect("arrow")
            outs = self.type_list()
        else:
            tys = [self.type_()]
            while self.accept("punct", ","):
                tys.append(self.type_())
            outs = [tys[-1]]          # `select` prints predicate type, value type
        return Op(name, operands, outs, attrs, [])

    def opaque_op(self, name):
        """An operation of another dialect (sharding annotations and the like):
        its SSA operands and trailing type are kept, the rest is skipped."""
        operands, depth = [], 0
        while True:
            t = self.peek()
            if t[0] == "eof":
                raise ParseError(f"unterminated {name}")
            if depth == 0 and t == ("punct", ":"):
                break
            if t[0] == "punct" and t[1] in "({[<":
                depth += 1
            elif t[0] == "punct" and t[1] in ")}]>":
                depth -= 1
            elif t[0] == "ssa":
                operands.append(self.lookup(t[1]))
            self.next()
        self.next()
        if self.peek() == ("punct", "("):
            self.type_list()
            self.expect("arrow")
            outs = self.type_list()
        else:
            outs = [self.type_()]
        return Op(name, operands, outs, {}, [])

    def while_op(self):
        self.expect("punct", "(")
        names, inits = [], []
        while not self.accept("punct", ")"):
            names.append(self.expect("ssa")[1][1:])
            self.expect("punct", "=")
            inits.append(self.lookup(self.expect("ssa")[1]))
            self.accept("punct", ",")
        self.expect("punct", ":")
        types = [self.type_()]
        while self.accept("punct", ","):
            types.append(self.type_())
        if self.accept("id", "attributes"):
            self.attr_dict()
        self.expect("id", "cond")
        cond = self.region_block([(n, Value(t, name=n)) for n, t in zip(names, types)])
        self.expect("id", "do")
        body = self.region_block([(n, Value(t, name=n)) for n, t in zip(names, types)])
        return Op("stablehlo.while", inits, types, {}, [cond, body])

    def reduce_op(self):
        # stablehlo.reduce(%a init: %c)[, (%b init: %d)] [applies stablehlo.add] across
        #   dimensions = [d] : (..) -> ..  [reducer(%x: T, %y: T) (%z: T, %w: T) { ops }]
        ins, inits = [], []
        while self.accept("punct", "("):
            ins.append(self.lookup(self.expect("ssa")[1]))
            self.expect("id", "init")
            self.expect("punct", ":")
            inits.append(self.lookup(self.expect("ssa")[1]))
            self.expect("punct", ")")
            if not self.accept("punct", ","):
                break
        attrs = {}
        regions = []
        if self.accept("id", "applies"):
            attrs["body"] = self.expect("id")[1]
        self.expect("id", "across")
        self.expect("id", "dimensions")
        self.expect("punct", "=")
        attrs["dimensions"] = self.int_list()
        _, outs = self.fn_type()
        if self.accept("id", "reducer"):
            firsts, seconds = [], []
            while self.accept("punct", "("):
                pair = []
                while not self.accept("punct", ")"):
                    ref = self.expect("ssa")[1][1:]
                    self.expect("punct", ":")
                    pair.append((ref, Value(self.type_(), name=ref)))
                    self.accept("punct", ",")
                firsts.append(pair[0])
                seconds.append(pair[1])
            regions.append(self.region_block(firsts + seconds))
        return Op("stablehlo.reduce", ins + inits, outs, attrs, regions)


def _hash_fields(payload: str) -> dict:
    """`a = [1, 2], b = 3` -> {"a": [1, 2], "b": 3} (dialect attribute bodies)."""
    out = {}
    for m in re.finditer(r"(\w+)\s*=\s*(\[[^\]]*\]|-?\d+)", payload):
        v = m.group(2)
        out[m.group(1)] = [int(x) for x in v[1:-1].replace(",", " ").split()] if v[0] == "[" else int(v)
    return out


def parse_module(text: str) -> Module:
    return _Parser(text).parse()


# ------------------------------------------------------- attribute access ----

def walk_blocks(block):
    """The block and every block nested in its ops' regions."""
    yield block
    for op in block.ops:
        for r in op.regions:
            yield from walk_blocks(r)


def i64_list(op, key):
    v = op.attrs.get(key)
    if v is None and key == "broadcast_dimensions":
        v = op.attrs.get("dims")
    if v is None and key == "permutation":
        v = op.attrs.get("dims")
    if v is None:
        raise KeyError(f"{op.name} has no attribute {key}")
    return list(v)


def dot_dims(op):
    """(lhs_batch, rhs_batch, lhs_contract, rhs_contract) of a dot_general."""
    if "dot_dimension_numbers" in op.attrs:       # generic form
        f = op.attrs["dot_dimension_numbers"][1]
        return (f.get("lhs_batching_dimensions", []), f.get("rhs_batching_dimensions", []),
                f.get("lhs_contracting_dimensions", []), f.get("rhs_contracting_dimensions", []))
    lb, rb = op.attrs.get("batching_dims", ([], []))
    lc, rc = op.attrs.get("contracting_dims", ([], []))
    return list(lb), list(rb), list(lc), list(rc)


_NP_EL = {"i1": np.bool_, "i4": np.int8, "ui4": np.uint8, "i8": np.int8, "ui8": np.uint8,
          "i16": np.int16, "ui16": np.uint16, "i32": np.int32, "ui32": np.uint32,
          "i64": np.int64, "ui64": np.uint64, "f16": np.float16, "bf16": np.float32,
          "f32": np.float32, "f64": np.float64}


def np_dtype(el: str):
    """Host storage dtype of an element type (bf16 is held as rounded float32,
    4-bit integers in 8-bit storage)."""
    return _NP_EL[el]


def dense_to_np(attr, ty: TensorType) -> np.ndarray:
    """The payload of a `dense<...>` attribute as a host array of `ty`'s shape:
    a splat scalar, a nested list, or a hex blob (`"0x..."`, raw little-endian
    element bytes; bf16 as its 16-bit patterns)."""
    _, payload, _ = attr
    payload = payload.strip()
    dt = np_dtype(ty.el)
    if payload.startswith('"0x'):
        raw = bytes.fromhex(payload.strip('"')[2:])
        if ty.el == "bf16":
            bits = np.frombuffer(raw, np.uint16).astype(np.uint32) << 16
            arr = bits.view(np.float32)
        elif ty.el == "i1":
            arr = np.frombuffer(raw, np.uint8).astype(np.bool_)
        else:
            arr = np.frombuffer(raw, np.dtype(dt))
        if arr.size == 1:
            return np.full(ty.shape, arr[0], dt)
        return arr.reshape(ty.shape).astype(dt)
    toks = re.findall(r"0x[0-9A-Fa-f]+|[-+]?(?:\d+\.\d*|\.\d+|\d+)(?:[eE][-+]?\d+)?|true|false|[-+]?inf|nan", payload)

    def conv(t):
        if t in ("true", "false"):
            return t == "true"
        if t.lower().startswith("0x"):
            bits = int(t, 16)
            if ty.el == "bf16":
                return np.array([bits << 16], np.uint32).view(np.float32)[0]
            if ty.el == "f16":
                return np.array([bits], np.uint16).view(np.float16)[0]
            if ty.el == "f32":
                return np.array([bits], np.uint32).view(np.float32)[0]
            if ty.el == "f64":
                return np.array([bits], np.uint64).view(np.float64)[0]
            return bits
        return float(t) if ty.el in ("f16", "bf16", "f32", "f64") else int(t)

    vals = [conv(t) for t in toks]
    if len(vals) == 1:
        arr = np.full(ty.shape, vals[0], dt)
    else:
        arr = np.array(vals, dt).reshape(ty.shape)
    if ty.el == "bf16":
        from .packing import f32_to_bf16_bits
        arr = (f32_to_bf16_bits(arr).astype(np.uint32) << 16).view(np.float32).reshape(ty.shape)
    return arr
