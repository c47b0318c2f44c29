"""The engine surface the recognizer hangs off: compile a StableHLO module,
execute it on buffers (reference src/metaljax/engine.py:325, :385).

Only what the quantized-matmul path needs is here: `compile_program` parses
the module text, `execute` runs the packing prologue and then the program.
The PJRT plugin, buffer donation/aliasing and the trace cache of the reference
engine are outside this package.
"""

from __future__ import annotations

from . import qmm
from .interpreter import Interpreter, host


class Executable:
    def __init__(self, interp, name="main"):
        self.interp = interp
        self.name = name
        self.num_params = len(interp.main.body.args)
        self.num_outputs = len(interp.main.result_types)
        self.out_types = [t.el for t in interp.main.result_types]
        self.out_dims = [list(t.shape) for t in interp.main.result_types]
        self.donated_params = sorted(interp.donated_args)
        self.generation = 0                 # bumped whenever the rewrite set changes

    def invalidate_traces(self):
        self.generation += 1
        self.interp.invalidate_plans()


def compile_program(code, fmt="mlir", options=None) -> Executable:
    """`code`: StableHLO module text (str or UTF-8 bytes)."""
    if fmt not in ("mlir", "stablehlo"):
        raise ValueError(f"Unsupported program format {fmt!r}: module text only")
    if isinstance(code, (bytes, bytearray)):
        code = bytes(code).decode("utf-8")
    return Executable(Interpreter(code))


def execute(ex: Executable, buffers):
    """Run the program.  Recognized weights are packed against these buffers
    first (a no-op once the same buffers have been seen); if that changed the
    set of rewritten dots, anything cached around the old structure is dropped
    (reference engine.py:395-400)."""
    args = list(buffers)
    if qmm.ENABLED:
        if qmm.prologue(ex.interp, args):
            ex.invalidate_traces()
    return ex.interp.run(args)


def to_host(buf):
    """A result as (numpy array, element type); bf16 comes back as float32 values."""
    h = host(buf)
    return h.a, h.el
