"""Expert-indexed quantized matmul over packs the qmm recognizer built: the
gathered dispatch that replaces a dense per-expert product.

A dense mixture-of-experts layer multiplies every token by every expert and
masks; the gathered form multiplies each (token, expert) pair once:

    y[p] = x[tidx[p]] . dequant(W[eidx[p]])^T        p in [0, P = T*K)

followed by the routing-weighted sum over each token's K experts.  This module
is the run-time half (reference src/metaljax/moe.py:1276-1340, :1425-1461):
`split_experts` re-views a pack with a leading expert axis, `emit_dot` issues
the expert-indexed product, `combine` weights and sums.  The pairs arrive in
token-major order, not sorted by expert; the library sorts rows by expert on
the device and runs the grouped kernel.  The graph-side planner that proves a
dense dispatch equivalent to this form is not part of this module.
"""

from __future__ import annotations

import os

MOE_ENABLED = os.environ.get("METALJAX_MOE", "1") != "0"
STATS = {"gather_qmm": 0, "dispatches": 0}


def stats() -> dict:
    return dict(STATS)


def reset_stats():
    for k in STATS:
        STATS[k] = 0


class Dot:
    """One expert product of a dispatch: the qmm match whose pack it reads
    (marked `absorbed`, so no dense quantized_matmul is emitted for it)."""

    def __init__(self, match):
        self.match = match
        match.absorbed = True


def split_experts(arrays, e):
    """Packed arrays [B.., N, ...] whose leading dims multiply to `e` expert
    slots, viewed as [E, N, ...] (reference moe.py:1276-1280)."""
    out = []
    for a in arrays:
        out.append(a.reshape((e,) + tuple(a.shape[-2:])))
    return out


def pair_indices(indices):
    """(tidx, eidx) for top-k `indices` [T, K]: pair p = t*K + j reads token t
    and expert indices[t, j] (reference moe.py:1295-1306, :1432-1433)."""
    import torch
    t, k = indices.shape
    tidx = torch.arange(t, device=indices.device, dtype=torch.int32).repeat_interleave(k)
    eidx = indices.reshape(t * k).to(torch.int32)
    return tidx, eidx


def emit_dot(x, arrays, mode, gs, bits, tidx, eidx, experts, out_dtype=None, has_perm=False):
    """y[p] = x[tidx[p]] . dequant(W[eidx[p]])^T -> [P, N]
    (reference moe.py:1283-1340, the mx.gather_qmm call at :1320).
    `arrays` are a pack's arrays (w, scales[, biases][, perm]) with the expert
    axis leading; `x` is [T, K] (or [P, K] with tidx None).  A pack built over
    a permuted contraction axis carries the permutation last: the activations
    are gathered through it first (reference moe.py:1316-1317)."""
    from . import kernels
    w, scales = arrays[0], arrays[1]
    biases = arrays[2] if mode == "affine" else None
    if has_perm:
        x = kernels.take_k(x, arrays[-1])
    w, scales = split_experts([w, scales], experts)
    if biases is not None:
        (biases,) = split_experts([biases], experts)
    STATS["gather_qmm"] += 1
    return kernels.gather_qmm(x, w, scales, biases, lhs_indices=tidx, rhs_indices=eidx,
                              group_size=gs, bits=bits, mode=mode, out_dtype=out_dtype)


def combine(y_pairs, weights):
    """Routing-weighted sum over each token's K experts: y_pairs [T*K, N],
    weights [T, K] -> [T, N] (reference moe.py:1444-1461)."""
    t, k = weights.shape
    y = y_pairs.reshape(t, k, -1).float() * weights.reshape(t, k, 1).float()
    return y.sum(dim=1).to(y_pairs.dtype)


def expert_dispatch(interp, match, x, indices, weights):
    """The whole gathered layer for one absorbed qmm match: pack lookup,
    expert-indexed product, weighted sum."""
    from . import qmm
    arrays = qmm.pack_arrays(interp, match)
    experts = 1
    for d in match.bshape:
        experts *= d
    tidx, eidx = pair_indices(indices)
    y = emit_dot(x, arrays, match.mode, match.gs, match.bits, tidx, eidx, experts,
                 out_dtype=qmm._torch_dtype(match.out_dtype), has_perm=match.has_perm)
    STATS["dispatches"] += 1
    return combine(y, weights)


# -- recognizer hooks shared with qmm's root dispatch.  No graph-side planner
# builds moe matches in this package, so these are only reached by a caller
# that registers one in State.moe itself.

def emit_reads(g):
    return tuple(g.reads)


def emit_bytes(g) -> int:
    return int(getattr(g, "bytes", 0))


def emit(interp, g, env):
    return g.run(interp, env)


def plan_dispatches(interp, st):
    return []
