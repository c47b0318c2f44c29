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

This module is the surface the interpreter and the engine call; the structural
matcher lives in `recognize.py`, evaluation / verification / packing and the
pack caches in `packs.py`.  What differs from the reference is below the
boundary: the fused op is `metaljax_amd.kernels.quantized_matmul`
(libqmm_hip.so through ctypes) on device tensors, and packing runs in numpy on
the host.  A missing library or GPU is an error at `emit`, never a silent
literal run.
"""

from __future__ import annotations

import os

import numpy as np

from . import ir, packing, packs, recognize
from .interpreter import host
from .packing import Reject
from .packs import Pack as _Pack                      # noqa: F401  (the reference's name for it)
from .packs import _BUILT, _SHARED, STATS             # noqa: F401  (tests clear / read these)
from .packs import evaluate as _eval                  # noqa: F401
from .recognize import Match

QMM_ENABLED = os.environ.get("METALJAX_QMM", "1") != "0"
ENABLED = QMM_ENABLED or os.environ.get("METALJAX_MOE", "1") != "0"
_DEBUG = os.environ.get("METALJAX_DEBUG", "") == "1"
# Row-blocked pack builds between two reclaims in `prologue` (a build that
# evaluated its weight whole reclaims at once; reference qmm.py:165).
GC_EVERY = int(os.environ.get("METALJAX_QMM_GC_EVERY", "8"))
RECLAIMS = [0]                          # reclaims made (tests count them)
_Reject = Reject


def _debug(msg):
    if _DEBUG:
        print(f"[metaljax_amd] qmm: {msg}", flush=True)


packs._debug = _debug


def stats() -> dict:
    return dict(STATS)


def reset_stats():
    for k in STATS:
        STATS[k] = 0


class State:
    """What one program's recognizer knows (reference qmm.py:667-699): its
    matches, and derived from the live ones the rewrite the interpreter
    applies -- `roots` (op key -> what replaces it), `skip` (keys of ops that
    never run) -- plus `values`, the packed arrays of the last prologue in slot
    order."""

    def __init__(self):
        self.matches = []
        self.moe = []                      # expert dispatches (metaljax_amd.moe)
        self.roots = {}
        self.skip = frozenset()
        self.values = []
        self.active = False

    def rebuild(self):
        roots, skipped = {}, set()
        for m in self.matches:
            if m.disabled:
                continue
            skipped.update(m.ops)
            if not m.absorbed:                  # an absorbed match emits nothing itself
                roots[m.key] = m
        for dispatch in self.moe:
            if not dispatch.disabled:
                roots[dispatch.key] = dispatch
                skipped.update(dispatch.skip_keys)
        self.roots, self.skip = roots, frozenset(skipped)
        self.active = bool(roots)


def analyze(interp) -> State:
    """Structural analysis of a program, once per interpreter; never looks at
    values and never fails the program: whatever goes wrong, the program runs
    literally (reference qmm.py:1042-1091)."""
    if interp._qmm is not None:
        return interp._qmm
    st = interp._qmm = State()
    if QMM_ENABLED:
        try:
            st.matches = recognize.find_matches(interp, _debug)
        except Exception as e:
            _debug(f"analysis failed ({e})")
            st.matches = []
    STATS["recognized"] += len(st.matches)
    if st.matches:
        _debug(f"{len(st.matches)} quantized matmul(s) recognized")
    if st.matches:
        try:
            from . import moe
            moe.analyze(interp, st)             # (nothing when moe.ENABLED is off)
        except Exception as e:                  # like the matcher: never fails the program
            _debug(f"expert-dispatch analysis failed ({e})")
            st.moe = []
    st.rebuild()
    interp.invalidate_plans()
    return st


def _kernel_limits(m):
    """Refuse before packing what the library would refuse at every step
    (its index ranges), so that such a dot runs literally from the start."""
    terms = {"f32": 3, "f16": 2}.get(m.act_dtype, 1)
    if m.B > 65535:
        raise Reject(f"{m.B} batch entries: more than the kernels' grid takes")
    if terms * m.B * m.M * m.K >= 1 << 30:
        raise Reject("the activations exceed the kernels' 32-bit index range")
    if m.N >= 1 << 31 or m.K >= 1 << 31 or m.N * (m.K // 2) >= 1 << 40:
        raise Reject("the weight exceeds the kernels' index range")


def _device_failure(err) -> bool:
    """Is this exception the device failing (a HIP error reported by the
    library, a torch accelerator error) rather than a weight that does not
    verify or pack?  Such an error must reach the caller: disabling the match
    would run the program literally and hide it."""
    from ._lib import QmmError
    if isinstance(err, QmmError) and getattr(err, "code", 0) == 5:
        return True
    name = type(err).__name__
    if name in ("AcceleratorError", "OutOfMemoryError"):
        return True
    return isinstance(err, RuntimeError) and ("HIP error" in str(err) or "CUDA error" in str(err))


def prologue(interp, args) -> bool:
    """Make sure every live match has a pack for exactly these argument
    buffers (packing eagerly what is new) and lay the packed arrays out in
    `values`.  A match whose weight cannot be verified or packed is disabled
    and runs literally from now on.  Returns True when the rewrite changed --
    a match was disabled, or a repack changed the kernel a match calls --
    (reference qmm.py:2305-2387)."""
    st = interp._qmm or analyze(interp)
    if not (st.matches or st.moe):
        return False
    from ._lib import QmmLibraryError
    rewrite_changed = False
    layout = []
    built = since_reclaim = 0
    for m in st.matches:
        if m.disabled:
            continue
        try:
            before = STATS["packs"]
            pk = packs.pack_for(interp, m, args, _kernel_limits)
            if STATS["packs"] != before:
                # A fresh build ran the weight's reconstruction at (a block
                # of) its full size: what that left behind is given back
                # before the next one adds to it, not after a prologue full of
                # them (reference qmm.py:2326-2347).
                built += 1
                since_reclaim += 1
                if not pk.blocked or since_reclaim >= GC_EVERY:
                    since_reclaim = 0
                    reclaim()
        except QmmLibraryError:
            raise                               # a missing library is an error, not a fallback
        except Exception as why:
            if _device_failure(why):
                raise                           # a failing device is an error too: the literal chain would hide it
            m.disabled = rewrite_changed = True
            STATS["fallbacks"] += 1
            _debug(f"{m.name} falls back to the literal chain ({why})")
            continue
        calls = (pk.mode, pk.gs, pk.bits, pk.perm is not None)
        if calls != (m.mode, m.gs, m.bits, m.has_perm):
            if m.gs:                            # not the first pack: the call itself changes
                rewrite_changed = True
            m.mode, m.gs, m.bits, m.has_perm = calls
        arrays = pk.arrays()
        m.slot, m.nvals = len(layout), len(arrays)
        layout += arrays
    if st.moe:
        from . import moe
        if moe.prologue(interp, st):            # a dispatch whose weight did not pack, or that fails its check, runs densely
            rewrite_changed = True
    if rewrite_changed:
        st.rebuild()
        interp.invalidate_plans()
    st.values = layout
    if built:
        reclaim()                               # also the tail of the blocked builds that skipped theirs
    return rewrite_changed


def reclaim():
    """Give back what pack builds leave behind: reference cycles among the
    evaluation's dead float32 intermediates (host memory the reference counts
    alone do not free), then the device blocks torch's allocator caches from
    the uploads' staging (reference qmm.py:2345-2347, :2382-2386:
    gc.collect() + mx.clear_cache())."""
    import gc
    gc.collect()
    RECLAIMS[0] += 1
    import torch
    if torch.cuda.is_available() and torch.cuda.is_initialized():
        torch.cuda.empty_cache()


# --------------------------------------------------------------------------
# runtime
# --------------------------------------------------------------------------

def values(interp):
    """The packed arrays of the last prologue, in slot order: the explicit
    trailing inputs of anything traced around the program."""
    st = getattr(interp, "_qmm", None)
    return () if st is None else st.values


def push(interp, vals):
    """Bind other arrays to the slots for the duration of a nested run (a
    traced function receives them as its trailing inputs).  Returns what `pop`
    restores, None when the program has no packed arrays."""
    st = getattr(interp, "_qmm", None)
    if st is None or not st.values:
        return None
    saved, st.values = st.values, list(vals)
    return (saved,)


def pop(interp, token):
    if token is not None:
        (interp._qmm.values,) = token


def pack_arrays(interp, m):
    """Match `m`'s arrays (w, scales[, biases][, perm]) out of the slots."""
    return interp._qmm.values[m.slot:m.slot + m.nvals]


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


def _torch_dtype(el):
    import torch
    return {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[el]


# Where the tensors of the fused calls and of a running expert dispatch live.
# The kernels take nothing else; the dispatch's tensor program between its
# kernel calls is plain torch, which is how its tests run it without a GPU.
DEVICE = "cuda"


def to_device(v):
    """A runtime value as a device tensor (bf16 HostArrays become bfloat16)."""
    import torch
    if isinstance(v, torch.Tensor):
        return v if v.device.type == DEVICE else v.to(DEVICE)
    h = host(v)
    if h.el == "bf16":
        bits = packing.f32_to_bf16_bits(h.a).view(np.int16)
        return torch.from_numpy(np.ascontiguousarray(bits)).to(DEVICE).view(torch.bfloat16)
    a = np.ascontiguousarray(h.a)
    if not a.flags.writeable:                   # torch refuses to wrap read-only storage without a warning
        a = a.copy()
    return torch.from_numpy(a).to(DEVICE)


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
    flat = [m.B, m.M, m.K] if m.bshape else [m.M, m.K]
    if list(x.shape) != flat:
        x = x.reshape(flat)
    if not x.is_contiguous():
        x = x.contiguous()
    if m.has_perm:
        x = kernels.take_k(x, vals[-1])
    y = kernels.quantized_matmul(x, w, scales, biases, transpose=True, group_size=m.gs,
                                 bits=m.bits, mode=m.mode, out_dtype=_torch_dtype(m.out_dtype))
    if m.swapped:
        y = y.transpose(-1, -2).reshape(m.bshape + m.nshape + m.mshape)
    else:
        shape = m.bshape + m.mshape + m.nshape
        if list(y.shape) != shape:
            y = y.reshape(shape)
    return [y]
