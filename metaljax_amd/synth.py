"""Seeded synthetic inputs of the named benchmark shapes.

Five workloads: decode GEMV (C1), small-batch int4 (C2), int8 prefill GEMM
(C3), MXFP4 GEMM (C4) and the quantized MoE grouped product (C5).  Every draw
comes from `np.random.default_rng(1000 + cfg)` in the order x, codes,
scales / exponents, router logits; float32 draws are rounded to bf16.  Arrays
are numpy (bf16 as uint16 bit patterns) so the same inputs feed the GPU path,
the tests and the CPU baseline.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

from .packing import f32_to_bf16_bits, pack_codes


@dataclass
class Workload:
    name: str
    cfg: int
    mode: str                 # "affine" | "mxfp4"
    bits: int
    group_size: int
    M: int
    N: int
    K: int
    E: int = 1                # experts (C5)
    x: np.ndarray = None      # bf16 bits [M, K]
    w: np.ndarray = None      # uint32 [(E,) N, K*bits/32]
    scales: np.ndarray = None  # bf16 bits [(E,) N, K/gs] or uint8 E8M0 [N, K/32]
    biases: np.ndarray = None
    row_offsets: np.ndarray = None   # int32 [E+1] (C5)
    extras: dict = field(default_factory=dict)

    @property
    def flops(self) -> int:
        return 2 * self.M * self.N * self.K

    @property
    def algorithmic_bytes(self) -> int:
        """Packed weight + tables + x + y, each counted once (y bf16)."""
        tot = self.w.nbytes + self.scales.nbytes + self.x.nbytes + self.M * self.N * 2
        if self.biases is not None:
            tot += self.biases.nbytes
        return int(tot)


SHAPES = {
    1: dict(name="C1 decode GEMV int4 g64", mode="affine", bits=4, M=1, N=4096, K=4096),
    2: dict(name="C2 small-batch int4 g64", mode="affine", bits=4, M=16, N=14336, K=4096),
    3: dict(name="C3 prefill GEMM int8 g64", mode="affine", bits=8, M=2048, N=4096, K=4096),
    4: dict(name="C4 mxfp4 GEMM", mode="mxfp4", bits=4, M=256, N=8192, K=8192),
    5: dict(name="C5 MoE grouped int4 g64", mode="affine", bits=4, M=1024, N=14336, K=4096, E=8),
}


def _bf16(x):
    return f32_to_bf16_bits(np.asarray(x, np.float32))


def make(cfg: int, scale: float = 1.0, M: int | None = None) -> Workload:
    """Build workload `cfg` (1-5).  `scale` < 1 shrinks N (and the token count
    of C5) for CPU-checkable parity cases; `M` overrides the activation rows."""
    sh = dict(SHAPES[cfg])
    rng = np.random.default_rng(1000 + cfg)
    n = max(16, int(sh["N"] * scale) // 16 * 16)
    k = sh["K"]
    m = sh["M"] if M is None else M
    e = sh.get("E", 1)
    bits, mode = sh["bits"], sh["mode"]
    wl = Workload(name=sh["name"], cfg=cfg, mode=mode, bits=bits,
                  group_size=32 if mode == "mxfp4" else 64, M=m, N=n, K=k, E=e)
    if cfg == 5:
        tokens = max(8, int(512 * scale)) if M is None else M // 2
        xt = _bf16(rng.standard_normal((tokens, k)))
    else:
        wl.x = _bf16(rng.standard_normal((m, k)))
    lead = (e,) if cfg == 5 else ()
    if mode == "affine":
        codes = rng.integers(0, 1 << bits, size=lead + (n, k), dtype=np.uint8)
        wl.w = pack_codes(codes, bits)
        del codes
        lo, hi = (0.005, 0.02) if bits == 4 else (0.0005, 0.002)
        s_bits = _bf16(rng.uniform(lo, hi, size=lead + (n, k // 64)))
        s = (s_bits.astype(np.uint32) << 16).view(np.float32)
        wl.scales = s_bits
        wl.biases = _bf16(-float(1 << (bits - 1)) * s)      # exact: a power-of-two multiple
    else:
        codes = rng.integers(0, 16, size=(n, k), dtype=np.uint8)
        wl.w = pack_codes(codes, 4)
        del codes
        wl.scales = rng.integers(120, 131, size=(n, k // 32)).astype(np.uint8)
        wl.biases = None
    if cfg == 5:
        logits = rng.standard_normal((tokens, e))
        p = np.exp(logits - logits.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        top = np.argsort(-p, axis=-1, kind="stable")[:, :2]          # [tokens, 2]
        flat = top.reshape(-1)
        order = np.argsort(flat, kind="stable")
        tok = (order // 2).astype(np.int32)
        wl.x = np.ascontiguousarray(xt[tok])
        wl.M = wl.x.shape[0]
        sizes = np.bincount(flat, minlength=e)
        wl.row_offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
        wl.extras = dict(tokens=tokens, token_of_row=tok, pair_of_row=order.astype(np.int32),
                         experts=top.astype(np.int32),
                         gates=np.take_along_axis(p, top, -1).astype(np.float32), x_tokens=xt)
    return wl


def to_device(wl: Workload, device="cuda"):
    """Torch tensors on `device`: (x bf16, w int32 view of the words, scales, biases, row_offsets)."""
    import torch
    def bf(a):
        return torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)
    x = bf(wl.x)
    w = torch.from_numpy(wl.w.view(np.int32)).to(device)
    if wl.mode == "affine":
        s, b = bf(wl.scales), bf(wl.biases)
    else:
        s, b = torch.from_numpy(wl.scales).to(device), None
    ro = None if wl.row_offsets is None else torch.from_numpy(wl.row_offsets).to(device)
    return x, w, s, b, ro


def affine_program_text(m: int, n: int, k: int, group_size: int = 64, el: str = "bf16") -> str:
    """A StableHLO module whose one dot the recognizer rewrites into the fused
    call: signed 4-bit-range codes i8 [N, K] viewed by groups, one scale and
    one zero point per group, `x @ ((q - z) * s)^T` (the sub-channel form of
    reference tests/test_qmm.py:991-1027).  Arguments: q i8 [N, K], scale
    [N, K/gs] (`el`), zero i8 [N, K/gs], x [M, K]; result [M, N]."""
    ng = k // group_size

    def t(shape, e):
        return "tensor<" + "x".join([*map(str, shape), e]) + ">"
    s3, q3 = t((n, ng, group_size), el), t((n, ng, group_size), "i8")
    return f"""
module @jit_affine_grouped {{
  func.func public @main(%q: {t((n, k), "i8")}, %scale: {t((n, ng), el)}, %zero: {t((n, ng), "i8")}, %x: {t((m, k), el)}) -> {t((m, n), el)} {{
    %qs = stablehlo.reshape %q : ({t((n, k), "i8")}) -> {q3}
    %qf = stablehlo.convert %qs : ({q3}) -> {s3}
    %sb = stablehlo.broadcast_in_dim %scale, dims = [0, 1] : ({t((n, ng), el)}) -> {s3}
    %zc = stablehlo.convert %zero : ({t((n, ng), "i8")}) -> {t((n, ng), el)}
    %zb = stablehlo.broadcast_in_dim %zc, dims = [0, 1] : ({t((n, ng), el)}) -> {s3}
    %d = stablehlo.subtract %qf, %zb : {s3}
    %w3 = stablehlo.multiply %d, %sb : {s3}
    %w = stablehlo.reshape %w3 : ({s3}) -> {t((n, k), el)}
    %y = stablehlo.dot_general %x, %w, contracting_dims = [1] x [1] : ({t((m, k), el)}, {t((n, k), el)}) -> {t((m, n), el)}
    return %y : {t((m, n), el)}
  }}
}}
"""
