"""Checkpoint-side producers: quantized weights as they sit in a checkpoint ->
the arrays the kernels read, with as little repacking as the format allows.

Two formats the reference meets:

* **HF MXFP4** (`*_blocks` uint8 `[..., out, K/32, 16]`, `*_scales` uint8
  `[..., out, K/32]`), loaded by the reference straight into packed variables
  (reference scripts/model_bench/mxfp4_gpt_oss.py:211-258): byte j of a block
  holds element 2j in its low nibble and 2j+1 in its high nibble, which is the
  LSB-first order of the packed uint32 stream (reference
  scripts/model_bench/mxfp4_gpt_oss.py:91-98), and the scale bytes are E8M0
  with bias 127.  Flattening the last two axes *is* the kernel layout: no copy.
* **keras int4** (`kernel` int8 `[K, N/2]`: the low nibble of byte j of a row is
  output column 2j, the high nibble column 2j+1, two's-complement nibbles;
  reference tests/test_qmm.py:179-190).  The kernels contract along K with K
  fastest, so this one is a real repack: unpack, flip the sign bit (code + 8),
  transpose, pack.

Nothing here touches the GPU except `to_device`.
"""

from __future__ import annotations

import numpy as np

from . import packing

MXFP4_BLOCK = 32                                 # values per E8M0 scale
_BLOCK_BYTES = MXFP4_BLOCK // 2


class CheckpointFormatError(ValueError):
    """The tensors do not have the layout this producer understands."""


def check_scale_range(scale_bytes, what: str = "") -> None:
    """E8M0 bytes 0 (2^-127, subnormal) and 255 (NaN) never occur in a real
    checkpoint; fail loudly rather than let one through (reference
    scripts/model_bench/mxfp4_gpt_oss.py:83-88)."""
    a = np.asarray(scale_bytes)
    if a.size == 0:
        return
    lo, hi = int(a.min()), int(a.max())
    if lo < 1 or hi > 254:
        raise CheckpointFormatError(
            f"{what}: E8M0 bytes span [{lo}, {hi}]; 0 and 255 are not usable scales")


def mxfp4_from_hf_blocks(blocks, scales, what: str = "mxfp4"):
    """HF `_blocks` / `_scales` -> (codes uint8 [..., N, K/2], scale bytes uint8
    [..., N, K/32]), both views of the inputs.

    `blocks` is uint8 `[..., N, K/32, 16]` (or already flat `[..., N, K/2]`),
    `scales` uint8 `[..., N, K/32]`; numpy arrays or torch tensors.  The codes
    array is what `kernels.quantized_matmul(..., mode="mxfp4")` takes as `w`
    (its uint8 form) and the scale bytes what it takes as `scales`.
    """
    if str(blocks.dtype).split(".")[-1] != "uint8" or str(scales.dtype).split(".")[-1] != "uint8":
        raise CheckpointFormatError(f"{what}: blocks and scales must be uint8, got "
                                    f"{blocks.dtype} / {scales.dtype}")
    bshape, sshape = tuple(blocks.shape), tuple(scales.shape)
    if len(bshape) == len(sshape) + 1:
        if bshape[-1] != _BLOCK_BYTES or bshape[:-1] != sshape:
            raise CheckpointFormatError(
                f"{what}: blocks {bshape} do not pair with scales {sshape} "
                f"(want [..., N, K/32, {_BLOCK_BYTES}] and [..., N, K/32])")
        codes = blocks.reshape(bshape[:-2] + (bshape[-2] * _BLOCK_BYTES,))
    elif len(bshape) == len(sshape):
        if bshape[:-1] != sshape[:-1] or bshape[-1] != sshape[-1] * _BLOCK_BYTES:
            raise CheckpointFormatError(
                f"{what}: flat codes {bshape} do not pair with scales {sshape}")
        codes = blocks
    else:
        raise CheckpointFormatError(f"{what}: blocks {bshape} vs scales {sshape}")
    host = scales.detach().cpu().numpy() if hasattr(scales, "detach") else scales
    check_scale_range(host, what)
    return codes, scales


def load_mxfp4_safetensors(path: str, blocks_key: str, scales_key: str):
    """Read one MXFP4 weight from a safetensors file (numpy, zero-copy views of
    the mapped file where safetensors allows it) and hand it over in kernel
    layout.  Nothing in the file is executed."""
    from safetensors import safe_open

    with safe_open(path, framework="np") as f:
        keys = set(f.keys())
        for k in (blocks_key, scales_key):
            if k not in keys:
                raise CheckpointFormatError(f"{path}: no tensor named {k!r}")
        blocks = f.get_tensor(blocks_key)
        scales = f.get_tensor(scales_key)
    return mxfp4_from_hf_blocks(blocks, scales, what=blocks_key)


def keras_int4_unpack(packed, columns: int) -> np.ndarray:
    """`keras.quantizers.unpack_int4` for the packed (axis=-1) layout as the
    reference restates it (reference tests/test_qmm.py:179-190): int8
    `[rows, ceil(columns/2)]` -> signed int8 `[rows, columns]` in [-8, 7]."""
    p = np.asarray(packed).view(np.uint8)
    low = (p & 15).astype(np.int8)
    high = (p >> 4).astype(np.int8)
    both = np.stack([low, high], axis=-1).reshape(p.shape[0], -1)[:, :columns]
    return ((both ^ 8) - 8).astype(np.int8)


def keras_int4_kernel_to_packed(packed, columns: int):
    """keras Dense int4 `kernel` `[K, N/2]` -> (uint32 words `[N, K/8]`, offset).

    The words hold the unsigned codes `q + 8`; `offset` (= 8) is what
    `packing.pack_exact` / `scale_bias` fold into the bias so that
    `scale * (code - 8 - zero)` is reproduced exactly
    (reference src/metaljax/qmm.py:235-282).
    """
    signed = keras_int4_unpack(packed, columns)          # [K, N]
    k = signed.shape[0]
    if k % 8:
        raise CheckpointFormatError(f"K = {k} is not a multiple of 8")
    codes = (signed.astype(np.int16) + 8).astype(np.uint8).T   # [N, K], 0..15
    return packing.pack_codes(np.ascontiguousarray(codes), 4), 8


def to_device(array, device="cuda"):
    """numpy -> torch on `device` (uint32 words travel as int32 bit patterns)."""
    import torch

    a = np.ascontiguousarray(array)
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    return torch.from_numpy(a).to(device)
