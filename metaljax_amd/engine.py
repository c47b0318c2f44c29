"""The engine surface the recognizer hangs off: compile a StableHLO module,
execute it on buffers (reference src/metaljax/engine.py:325, :385).

Only what the quantized-matmul path needs is here: `compile_program` parses
the module text, `execute` runs the packing prologue and then the program.
Buffer donation/aliasing and the trace cache of the reference engine are
outside this package.  What a PJRT plugin calls by name (csrc/pjrt_plugin.cc
is one) keeps its name,
argument meaning and result type (reference plugin/metal_pjrt.cc):

    compile_program(code, fmt, options) -> object with name, fingerprint,
        num_outputs, num_params, out_types (PJRT_Buffer_Type integers),
        out_dims, donated_params                       metal_pjrt.cc:547-580
    execute(executable, [buffer]) -> [buffer]; a buffer has data, type_enum,
        dims, nbytes                                   metal_pjrt.cc:284-299, :990-1010
    buffer_from_host(memoryview, type_enum, dims, byte_strides, offset)
                                                       metal_pjrt.cc:662-664
    to_host(buffer) -> bytes                           metal_pjrt.cc:1168-1172
    buffer_pointer(buffer) -> int                      metal_pjrt.cc:1125
    device_kind() -> str, stablehlo_version() -> [int] metal_pjrt.cc:382, :440

The reference's executables also carry `forwarded_outputs`-style donation
plumbing inside `execute`; here `donated_params` is reported, every output is
a fresh buffer, and the plugin drops a donated argument's buffer after the
call (csrc/pjrt_plugin.cc).
"""

from __future__ import annotations

import hashlib
import os

import numpy as np

from . import qmm
from .interpreter import HostArray, Interpreter, from_numpy, host
from .ir import np_dtype as ir_np_dtype

# PJRT_Buffer_Type enumerators, in the order of the PJRT C API
PJRT_TYPES = [
    "INVALID", "PRED", "S8", "S16", "S32", "S64", "U8", "U16", "U32", "U64",
    "F16", "F32", "F64", "BF16", "C64", "C128",
    "F8E5M2", "F8E4M3FN", "F8E4M3B11FNUZ", "F8E5M2FNUZ", "F8E4M3FNUZ",
    "S4", "U4", "TOKEN", "S2", "U2", "F8E4M3", "F8E3M4", "F8E8M0FNU",
    "F4E2M1FN", "S1", "U1", "F6E2M3FN", "F6E3M2FN",
]
_ENUM = {name: i for i, name in enumerate(PJRT_TYPES)}
# enumerator -> (StableHLO element type, numpy dtype of the host bytes)
_ENUM_EL = {
    _ENUM["PRED"]: ("i1", np.bool_), _ENUM["S8"]: ("i8", np.int8), _ENUM["S16"]: ("i16", np.int16),
    _ENUM["S32"]: ("i32", np.int32), _ENUM["S64"]: ("i64", np.int64), _ENUM["U8"]: ("ui8", np.uint8),
    _ENUM["U16"]: ("ui16", np.uint16), _ENUM["U32"]: ("ui32", np.uint32),
    _ENUM["U64"]: ("ui64", np.uint64), _ENUM["F16"]: ("f16", np.float16),
    _ENUM["F32"]: ("f32", np.float32), _ENUM["F64"]: ("f64", np.float64),
    _ENUM["BF16"]: ("bf16", np.uint16),          # host bytes are the 16-bit patterns
}
_EL_ENUM = {el: k for k, (el, _) in _ENUM_EL.items()}


class Buffer:
    """A runtime value plus the metadata a PJRT plugin reads: `data` (a host
    array or a device tensor), `type_enum`, `dims`, `nbytes`."""

    __slots__ = ("data", "type_enum", "dims", "nbytes")

    def __init__(self, data, type_enum: int, dims):
        self.data = data
        self.type_enum = int(type_enum)
        self.dims = [int(d) for d in dims]
        n = 1
        for d in self.dims:
            n *= d
        self.nbytes = n * np.dtype(_ENUM_EL[self.type_enum][1]).itemsize


def buffer_from_host(data, type_enum: int, dims, byte_strides=None, offset: int = 0) -> Buffer:
    """Host bytes (any buffer-protocol object, or None for zeros) -> Buffer.
    `byte_strides` / `offset` describe a strided view of `data`, as PJRT's
    BufferFromHostBuffer hands it over."""
    dims = [int(d) for d in dims]
    if type_enum not in _ENUM_EL:
        name = PJRT_TYPES[type_enum] if 0 <= type_enum < len(PJRT_TYPES) else type_enum
        raise TypeError(f"Unsupported PJRT buffer type {name}")
    el, dt = _ENUM_EL[type_enum]
    if data is None:
        arr = np.zeros(dims, dt)
    elif byte_strides is None:
        arr = np.frombuffer(data, dt).reshape(dims).copy()
    else:
        arr = np.ndarray(shape=dims, dtype=dt, buffer=data, offset=offset, strides=list(byte_strides))
        arr = np.array(arr, order="C", copy=True).reshape(dims)
    # (the bytes are copied either way: the caller's memory is free again when
    # this returns, which is what the plugin tells PJRT, pjrt_plugin.cc)
    if device_resident():
        return Buffer(_upload(arr, el), type_enum, dims)
    if el == "bf16":
        h = from_numpy((arr.astype(np.uint32) << 16).view(np.float32), el)   # held as float32 values
        h.bits = np.ascontiguousarray(arr)                                   # and as the type's own bytes
        return Buffer(h, type_enum, dims)
    return Buffer(from_numpy(arr, el), type_enum, dims)


def device_resident() -> bool:
    """Do buffers live on the GPU?  Yes whenever one is visible (the
    reference's `MetalBuffer.data` is a device array, engine.py:118-159);
    METALJAX_HOST_BUFFERS=1 keeps them on the host."""
    if os.environ.get("METALJAX_HOST_BUFFERS") == "1":
        return False
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def _upload(arr: np.ndarray, el: str):
    """Host bytes in the element type's own storage -> a device tensor of that
    type (bf16: the 16-bit patterns become a bfloat16 tensor)."""
    import torch
    arr = np.ascontiguousarray(arr)
    if el == "bf16":
        return torch.from_numpy(arr.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(arr).cuda()


def _resident(v, el):
    """A result value as what a Buffer of this engine holds: a device tensor
    when buffers are device-resident, the value itself otherwise."""
    if not isinstance(v, HostArray) or not device_resident():       # (a fused result is a device tensor already)
        return v
    if el == "bf16":
        from .packing import f32_to_bf16_bits
        return _upload(f32_to_bf16_bits(np.ascontiguousarray(v.a, np.float32)), "bf16")
    if el in ("i4", "ui4"):
        return v                                    # no 4-bit tensor type: stays a host array
    a = np.ascontiguousarray(v.a)
    if not a.flags.writeable:
        a = a.copy()
    return _upload(a, el)


def to_host(buf) -> bytes:
    """The bytes of a Buffer (or of any runtime value) in its element type,
    row-major (reference engine.py:154-159; what the plugin's ToHostBuffer
    copies out, metal_pjrt.cc:1168-1172)."""
    h = host(buf.data if isinstance(buf, Buffer) else buf)
    if h.el == "bf16":
        from .packing import f32_to_bf16_bits
        return f32_to_bf16_bits(np.ascontiguousarray(h.a, np.float32)).tobytes()
    return np.ascontiguousarray(h.a).tobytes()


buffer_to_host = to_host        # the name earlier callers of this package used


def to_numpy(buf):
    """A result as (numpy array, element type); bf16 comes back as float32 values."""
    h = host(buf.data if isinstance(buf, Buffer) else buf)
    return h.a, h.el


def buffer_pointer(buf) -> int:
    """Address of the value's storage: the device pointer of a tensor, the
    host address of a host array (stable while the Buffer is alive)."""
    v = buf.data if isinstance(buf, Buffer) else buf
    if isinstance(v, HostArray):
        if v.el == "bf16" and v.bits is not None:
            return int(v.bits.ctypes.data)
        if v.el == "bf16" or v.a.dtype != ir_np_dtype(v.el):
            # host bf16 values are held as float32: a reader of `nbytes` bytes
            # at this address would get something else than the advertised type
            raise UnsupportedProgram(f"Unsupported: a host-held {v.el} buffer has no storage in its own "
                                     "element type to point at")
        return int(v.a.ctypes.data)
    return int(v.data_ptr())


def device_kind() -> str:
    try:
        import torch
        if torch.cuda.is_available():
            return torch.cuda.get_device_name(0)
    except Exception:
        pass
    return "AMD GPU (none visible)"


def stablehlo_version() -> list:
    """The StableHLO text forms `ir.parse_module` reads are those of the 1.x
    pretty printer; there is no MLIR library to ask."""
    return [1, 0, 0]


class Executable:
    def __init__(self, interp, name="main", fingerprint=""):
        self.interp = interp
        self.name = name
        self.fingerprint = fingerprint
        self.num_params = len(interp.main.body.args)
        self.num_outputs = len(interp.main.result_types)
        # PJRT_Buffer_Type integers, as the plugin reads them (metal_pjrt.cc:558)
        unknown = [t.el for t in interp.main.result_types if t.el not in _EL_ENUM]
        if unknown:
            raise UnsupportedProgram(f"Unsupported result element type(s) {unknown}: no PJRT buffer type for them here")
        self.out_types = [_EL_ENUM[t.el] for t in interp.main.result_types]
        self.out_els = [t.el for t in interp.main.result_types]
        self.out_dims = [list(t.shape) for t in interp.main.result_types]
        self.donated_params = sorted(interp.donated_args)
        self.generation = 0                 # bumped whenever the rewrite set changes

    def invalidate_traces(self):
        self.generation += 1
        self.interp.invalidate_plans()


class UnsupportedProgram(ValueError):
    """A program this engine cannot read ("Unsupported" in the class name: a
    PJRT plugin reports it as UNIMPLEMENTED, reference metal_pjrt.cc:185-226)."""


_BYTECODE_MAGIC = b"ML\xefR"


def _module_text(raw: bytes) -> str:
    """Module text of what a client handed over.  A JAX client serialises the
    module as a StableHLO portable artifact (MLIR bytecode); this package reads
    text only, so the bytecode is printed back to text by the MLIR bindings
    that ship with jaxlib -- present wherever such a client runs, absent where
    this package was built (then: UnsupportedProgram)."""
    if not raw.startswith(_BYTECODE_MAGIC):
        return raw.decode("utf-8")
    try:
        from jaxlib.mlir import ir as mlir
        from jaxlib.mlir.dialects import stablehlo
    except Exception as e:
        raise UnsupportedProgram("MLIR bytecode needs jaxlib's MLIR bindings to be printed as text "
                                 f"(import failed: {e})") from None
    with mlir.Context() as ctx:
        stablehlo.register_dialect(ctx)
        try:
            module = stablehlo.deserialize_portable_artifact(ctx, raw)
        except Exception:
            module = mlir.Module.parse(raw, ctx)
        return module.operation.get_asm(enable_debug_info=False)


def compile_program(code, fmt="mlir", options=None) -> Executable:
    """`code`: a StableHLO module, as text (str or UTF-8 bytes) or as the MLIR
    bytecode a JAX client sends (see `_module_text`)."""
    if fmt not in ("mlir", "stablehlo"):
        raise UnsupportedProgram(f"Unsupported program format {fmt!r}: StableHLO modules only")
    raw = bytes(code) if isinstance(code, (bytes, bytearray, memoryview)) else code.encode("utf-8")
    return Executable(Interpreter(_module_text(raw)), fingerprint=hashlib.sha256(raw).hexdigest())


def execute(ex: Executable, buffers):
    """Run the program.  Recognized weights are packed against these buffers
    first (a no-op once the same buffers have been seen); if that changed the
    set of rewritten dots, anything cached around the old structure is dropped
    (reference engine.py:395-400)."""
    args = [b.data if isinstance(b, Buffer) else b for b in buffers]
    if qmm.ENABLED:
        if qmm.prologue(ex.interp, args):
            ex.invalidate_traces()
    outs = ex.interp.run(args)
    # every output as a buffer object (data, type_enum, dims, nbytes), which is
    # what the plugin wraps (metal_pjrt.cc:990-1010); `data` is a device tensor
    # whenever a GPU is visible (a literal op's host result is uploaded), as the
    # reference's buffers hold device arrays
    return [Buffer(_resident(v, el), t, d) for v, el, t, d in zip(outs, ex.out_els, ex.out_types, ex.out_dims)]
