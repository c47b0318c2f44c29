"""Torch-owned-buffer front end of the HIP library.

These functions are the drop-in for the three MLX calls the reference's
quantized path makes -- `mx.quantized_matmul` (reference
src/metaljax/qmm.py:2491), `mx.gather_qmm` (src/metaljax/moe.py:1320) and
`mx.dequantize` (tests only) -- with the same argument meaning.  PyTorch only
owns the device buffers and the stream; all arithmetic happens in
libqmm_hip.so.  Errors from the library surface as exceptions
(`UnsupportedQmm` when the combination is not built, so a caller can run the
literal chain, as the reference does on any packing or launch failure).
"""

from __future__ import annotations

import torch

from . import _lib
from ._lib import BF16, F16, F32, MODE_AFFINE, MODE_MXFP4, QmmError, UnsupportedQmm  # noqa: F401

_DT = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}
_MODE = {"affine": MODE_AFFINE, "mxfp4": MODE_MXFP4}


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


# One scratch allocation per (device, stream), grown to the largest request seen:
# calls on one stream are ordered, so the next call may overwrite what the
# previous one used; nothing is allocated per call once it has grown.  (A call
# recorded into a graph keeps the address it saw: record the Bound* forms below,
# which own their workspace for as long as they live, not these calls.)
_SCRATCH = {}


def _scratch(need: int, like: torch.Tensor):
    if not need:
        return None
    key = (like.device.index, _stream(like))
    ws = _SCRATCH.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(max(need, 1 << 16), dtype=torch.uint8, device=like.device)
        _SCRATCH[key] = ws
    return ws


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise _lib.QmmError(1, "tensors must live on the GPU (there is no CPU path)")


def _dt(t: torch.dtype) -> int:
    try:
        return _DT[t]
    except KeyError:
        raise UnsupportedQmm(3, f"dtype {t}") from None


def _ptr(t):
    return None if t is None else t.data_ptr()


def _weight_dims(w: torch.Tensor, bits: int, mode: str):
    """(lead dims, N, K) of a packed weight (uint32 words, or uint8 bytes)."""
    per = (8 // bits) if w.dtype == torch.uint8 else (32 // bits)
    if mode == "mxfp4":
        per = 2 if w.dtype == torch.uint8 else 8
    return tuple(w.shape[:-2]), w.shape[-2], w.shape[-1] * per


def quantized_matmul(x, w, scales, biases=None, transpose=True, group_size=64, bits=4,
                     mode="affine", out_dtype=None):
    """y[..., M, N] = x[..., M, K] @ dequant(w)[..., N, K]^T, float32 accumulate.

    x [M,K] or [B,M,K] (bf16, float16 or float32); w uint32 [(B,)N,K*bits/32] (or the same bytes
    as uint8); scales/biases [(B,)N,K/group_size] (bf16/f16/f32), for mxfp4
    uint8 E8M0 [(B,)N,K/32] and biases None.  Result dtype = out_dtype or x's.
    """
    if not transpose:
        raise UnsupportedQmm(3, "only transpose=True (weight stored [N, K]) is built")
    _need_cuda(x, w, scales, biases)
    lib = _lib.load()
    lead, n, k = _weight_dims(w, bits, mode)
    if x.shape[-1] != k:
        raise _lib.QmmError(2, f"x K={x.shape[-1]} vs weight K={k}")
    m = x.shape[-2]
    xlead = tuple(x.shape[:-2])
    if lead and xlead != lead:
        raise _lib.QmmError(2, f"batch dims {xlead} vs {lead}")
    batch = 1
    for d in lead:
        batch *= d
    x2 = x.contiguous()
    mrows = m
    if not lead:
        # unbatched weight: leading activation dims fold into M
        for d in xlead:
            mrows *= d
    out_dtype = out_dtype or x.dtype
    y = torch.empty(xlead + (m, n), dtype=out_dtype, device=x.device)
    w, scales = w.contiguous(), scales.contiguous()
    biases = None if biases is None else biases.contiguous()
    tab = _dt(scales.dtype) if mode == "affine" else BF16
    need = int(lib.qmm_workspace_bytes(batch, mrows, n, k, group_size, bits, _MODE[mode],
                                       _dt(x2.dtype)))
    ws = _scratch(need, x)
    rc = lib.qmm_quantized_matmul(
        _ptr(x2), _dt(x2.dtype), _ptr(w), _ptr(scales), _ptr(biases), tab, _ptr(y), _dt(out_dtype),
        batch, mrows, n, k, group_size, bits, _MODE[mode], _ptr(ws), need, _stream(x))
    _lib.check(rc)
    return y


def grouped_qmm(x, w, scales, biases, row_offsets, group_size=64, bits=4, mode="affine",
                out_dtype=None, out=None):
    """Rows of x [R,K] sorted by expert; rows [row_offsets[e], row_offsets[e+1])
    multiply expert e's weight w[e] ([E,N,...]).  row_offsets int32 [E+1] on the
    device.  Returns [R,N]: a new tensor whose rows outside the offsets are
    zero, or `out` (contiguous [R,N] of the output type), whose rows outside the
    offsets are left as they are."""
    _need_cuda(x, w, scales, biases, row_offsets)
    lib = _lib.load()
    (e,), n, k = _weight_dims(w, bits, mode)
    r = x.shape[0]
    if out is not None:
        _need_cuda(out)
        out_dtype = out_dtype or out.dtype
        if tuple(out.shape) != (r, n) or out.dtype != out_dtype or not out.is_contiguous():
            raise ValueError(f"out must be a contiguous [{r},{n}] tensor of {out_dtype}")
        y = out
    else:
        out_dtype = out_dtype or x.dtype
        y = torch.zeros((r, n), dtype=out_dtype, device=x.device)
    x, w, scales = x.contiguous(), w.contiguous(), scales.contiguous()
    biases = None if biases is None else biases.contiguous()
    ro = row_offsets.to(torch.int32).contiguous()
    tab = _dt(scales.dtype) if mode == "affine" else BF16
    need = int(lib.qmm_workspace_bytes(1, r, n, k, group_size, bits, _MODE[mode], _dt(x.dtype)))
    ws = _scratch(need, x)
    rc = lib.qmm_grouped_qmm(_ptr(x), _dt(x.dtype), _ptr(w), _ptr(scales), _ptr(biases), tab,
                             _ptr(y), _dt(out_dtype), _ptr(ro), r, e, n, k, group_size, bits,
                             _MODE[mode], _ptr(ws), need, _stream(x))
    _lib.check(rc)
    return y


def gather_qmm(x, w, scales, biases=None, lhs_indices=None, rhs_indices=None, transpose=True,
               group_size=64, bits=4, mode="affine", out_dtype=None):
    """y[p] = x[lhs_indices[p]] @ dequant(w[rhs_indices[p]])^T for every pair p.

    x [T,K] -> y [P,N], or x [T,M,K] (M activation rows per entry, as
    mx.gather_qmm takes it, reference src/metaljax/moe.py:1293-1301) ->
    y [P,M,N]; w [E,N,...]; indices int32 [P] in any order; lhs_indices None
    means pair p reads entry p.  With M rows per entry every pair becomes M
    one-row pairs of the same expert (rows lhs*M .. lhs*M + M - 1 of the
    flattened activations), which is what the library multiplies.
    """
    if not transpose:
        raise UnsupportedQmm(3, "only transpose=True is built")
    _need_cuda(x, w, scales, biases, lhs_indices, rhs_indices)
    lib = _lib.load()
    (e,), n, k = _weight_dims(w, bits, mode)
    rhs = rhs_indices.to(torch.int32).contiguous()
    lhs = None if lhs_indices is None else lhs_indices.to(torch.int32).contiguous()
    rows, with_rows = 1, x.dim() == 3
    if with_rows:
        rows = x.shape[1]
        x = x.reshape(x.shape[0] * rows, x.shape[2])
        if rows > 1:
            step = torch.arange(rows, device=rhs.device, dtype=torch.int32)
            first = (torch.arange(rhs.numel(), device=rhs.device, dtype=torch.int32) if lhs is None else lhs) * rows
            lhs = (first[:, None] + step[None, :]).reshape(-1).contiguous()
            rhs = rhs.repeat_interleave(rows).contiguous()
    elif x.dim() != 2:
        raise _lib.QmmError(2, f"x must be [T, K] or [T, M, K], got {tuple(x.shape)}")
    t = x.shape[0]
    p = rhs.numel()
    out_dtype = out_dtype or x.dtype
    y = torch.empty((p, n), dtype=out_dtype, device=x.device)
    x, w, scales = x.contiguous(), w.contiguous(), scales.contiguous()
    biases = None if biases is None else biases.contiguous()
    nbytes = int(lib.qmm_gather_workspace_bytes(p, e, n, k, _dt(x.dtype)))
    ws = _scratch(nbytes, x)
    tab = _dt(scales.dtype) if mode == "affine" else BF16
    rc = lib.qmm_gather_qmm(_ptr(x), _dt(x.dtype), _ptr(w), _ptr(scales), _ptr(biases), tab,
                            _ptr(y), _dt(out_dtype), _ptr(lhs), _ptr(rhs), p, t, e, n, k,
                            group_size, bits, _MODE[mode], _ptr(ws), nbytes, _stream(x))
    _lib.check(rc)
    return y.reshape(p // rows, rows, n) if with_rows else y


def dequantize(w, scales, biases=None, group_size=64, bits=4, mode="affine",
               out_dtype=torch.float32):
    """Packed weight -> [..., K] values (bit-exact fma / E2M1*2^e)."""
    _need_cuda(w, scales, biases)
    lib = _lib.load()
    lead, n, k = _weight_dims(w, bits, mode)
    rows = n
    for d in lead:
        rows *= d
    out = torch.empty(lead + (n, k), dtype=out_dtype, device=w.device)
    w, scales = w.contiguous(), scales.contiguous()
    biases = None if biases is None else biases.contiguous()
    tab = _dt(scales.dtype) if mode == "affine" else BF16
    rc = lib.qmm_dequantize(_ptr(w), _ptr(scales), _ptr(biases), tab, _ptr(out), _dt(out_dtype),
                            rows, k, group_size, bits, _MODE[mode], _stream(w))
    _lib.check(rc)
    return out


def unpack_codes(w, bits):
    """uint32 words [..., W] -> uint8 codes [..., W*32/bits]."""
    _need_cuda(w)
    lib = _lib.load()
    w = w.contiguous()
    k = w.shape[-1] * (32 // bits)
    rows = w.numel() // w.shape[-1] if w.numel() else 0
    out = torch.empty(tuple(w.shape[:-1]) + (k,), dtype=torch.uint8, device=w.device)
    _lib.check(lib.qmm_unpack_codes(_ptr(w), _ptr(out), rows, k, bits, _stream(w)))
    return out


def pack_codes(codes, bits):
    """uint8 codes [..., K] -> uint32 words [..., K*bits/32] (device-side)."""
    _need_cuda(codes)
    lib = _lib.load()
    codes = codes.to(torch.uint8).contiguous()
    k = codes.shape[-1]
    rows = codes.numel() // k if codes.numel() else 0
    out = torch.empty(tuple(codes.shape[:-1]) + (k * bits // 32,), dtype=torch.int32,
                      device=codes.device)
    _lib.check(lib.qmm_pack_codes(_ptr(codes), _ptr(out), rows, k, bits, _stream(codes)))
    return out


def take_k(x, perm):
    """x[..., perm] along the last axis (perm int32 [K] on the device)."""
    _need_cuda(x, perm)
    lib = _lib.load()
    x = x.contiguous()
    k = x.shape[-1]
    rows = x.numel() // k if x.numel() else 0
    out = torch.empty_like(x)
    perm = perm.to(torch.int32).contiguous()
    _lib.check(lib.qmm_take_k(_ptr(x), _dt(x.dtype), _ptr(perm), _ptr(out), rows, k, _stream(x)))
    return out


def plan(m, n, k, group_size=64, bits=4, mode="affine"):
    """(kernel family, grid, block) the dispatcher picks for a shape."""
    import ctypes
    lib = _lib.load()
    a, b, c = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    lib.qmm_plan(m, n, k, group_size, bits, _MODE[mode], ctypes.byref(a), ctypes.byref(b),
                 ctypes.byref(c))
    return a.value, b.value, c.value


class BoundQmm:
    """A quantized_matmul call with every argument resolved once.

    For launch-bound loops (decode steps, benchmarks, HIP-graph capture): the
    tensors are validated and kept alive here and `launch()` only issues the
    library call on the current stream into the preallocated `y`.
    """

    def __init__(self, x, w, scales, biases, y, group_size=64, bits=4, mode="affine"):
        _need_cuda(x, w, scales, biases, y)
        lead, n, k = _weight_dims(w, bits, mode)
        if lead or x.dim() != 2:
            raise UnsupportedQmm(3, "BoundQmm serves the unbatched [M,K] x [N,K] form")
        for t in (x, w, scales, biases, y):
            if t is not None and not t.is_contiguous():
                raise _lib.QmmError(1, "BoundQmm needs contiguous tensors")
        self._lib = _lib.load()
        tab = _dt(scales.dtype) if mode == "affine" else BF16
        need = int(self._lib.qmm_workspace_bytes(1, x.shape[0], n, k, group_size, bits,
                                                 _MODE[mode], _dt(x.dtype)))
        ws = torch.empty(need, dtype=torch.uint8, device=x.device) if need else None
        self._keep = (x, w, scales, biases, y, ws)
        self._args = (_ptr(x), _dt(x.dtype), _ptr(w), _ptr(scales), _ptr(biases), tab, _ptr(y),
                      _dt(y.dtype), 1, x.shape[0], n, k, group_size, bits, _MODE[mode], _ptr(ws),
                      need)
        self.y = y

    def launch(self, stream=None):
        st = stream if stream is not None else torch.cuda.current_stream().cuda_stream
        rc = self._lib.qmm_quantized_matmul(*self._args, st)
        if rc:
            _lib.check(rc)
        return self.y


class BoundGrouped:
    """A grouped_qmm call with every argument resolved once (see BoundQmm):
    rows of `x` sorted by expert, `row_offsets` int32 [E+1] on the device,
    results into the preallocated `y` (rows outside the offsets are left as
    they are)."""

    def __init__(self, x, w, scales, biases, row_offsets, y, group_size=64, bits=4, mode="affine"):
        _need_cuda(x, w, scales, biases, row_offsets, y)
        (e,), n, k = _weight_dims(w, bits, mode)
        for t in (x, w, scales, biases, row_offsets, y):
            if t is not None and not t.is_contiguous():
                raise _lib.QmmError(1, "BoundGrouped needs contiguous tensors")
        if row_offsets.dtype != torch.int32 or tuple(y.shape) != (x.shape[0], n):
            raise _lib.QmmError(1, "row_offsets must be int32 and y [rows, N]")
        self._lib = _lib.load()
        tab = _dt(scales.dtype) if mode == "affine" else BF16
        r = x.shape[0]
        need = int(self._lib.qmm_workspace_bytes(1, r, n, k, group_size, bits, _MODE[mode], _dt(x.dtype)))
        ws = torch.empty(need, dtype=torch.uint8, device=x.device) if need else None
        self._keep = (x, w, scales, biases, row_offsets, y, ws)
        self._args = (_ptr(x), _dt(x.dtype), _ptr(w), _ptr(scales), _ptr(biases), tab, _ptr(y),
                      _dt(y.dtype), _ptr(row_offsets), r, e, n, k, group_size, bits, _MODE[mode],
                      _ptr(ws), need)
        self.y = y

    def launch(self, stream=None):
        st = stream if stream is not None else torch.cuda.current_stream().cuda_stream
        rc = self._lib.qmm_grouped_qmm(*self._args, st)
        if rc:
            _lib.check(rc)
        return self.y


class BoundGather:
    """A gather_qmm call with every argument resolved once (see BoundQmm):
    x [T, K]; lhs / rhs indices int32 [P] on the device (pair p reads row
    lhs[p] of x and expert rhs[p]); results into the preallocated `y` [P, N]
    (a pair whose expert index is outside the weight leaves its row alone)."""

    def __init__(self, x, w, scales, biases, lhs_indices, rhs_indices, y, group_size=64, bits=4, mode="affine"):
        _need_cuda(x, w, scales, biases, lhs_indices, rhs_indices, y)
        (e,), n, k = _weight_dims(w, bits, mode)
        for t in (x, w, scales, biases, lhs_indices, rhs_indices, y):
            if t is not None and not t.is_contiguous():
                raise _lib.QmmError(1, "BoundGather needs contiguous tensors")
        p = rhs_indices.numel()
        if rhs_indices.dtype != torch.int32 or (lhs_indices is not None and lhs_indices.dtype != torch.int32):
            raise _lib.QmmError(1, "indices must be int32")
        if x.dim() != 2 or tuple(y.shape) != (p, n):
            raise _lib.QmmError(1, "x must be [T, K] and y [P, N]")
        self._lib = _lib.load()
        tab = _dt(scales.dtype) if mode == "affine" else BF16
        need = int(self._lib.qmm_gather_workspace_bytes(p, e, n, k, _dt(x.dtype)))
        ws = torch.empty(need, dtype=torch.uint8, device=x.device) if need else None
        self._keep = (x, w, scales, biases, lhs_indices, rhs_indices, y, ws)
        self._args = (_ptr(x), _dt(x.dtype), _ptr(w), _ptr(scales), _ptr(biases), tab, _ptr(y),
                      _dt(y.dtype), _ptr(lhs_indices), _ptr(rhs_indices), p, x.shape[0], e, n, k,
                      group_size, bits, _MODE[mode], _ptr(ws), need)
        self.y = y

    def launch(self, stream=None):
        st = stream if stream is not None else torch.cuda.current_stream().cuda_stream
        rc = self._lib.qmm_gather_qmm(*self._args, st)
        if rc:
            _lib.check(rc)
        return self.y
