"""Checkpoint-side producers against the oracle (no GPU).

HF MXFP4 blocks: the reference loads `_blocks` / `_scales` into packed variables
with a reshape only (reference scripts/model_bench/mxfp4_gpt_oss.py:211-258) and
dequantizes them as `E2M1[nibble] * 2**(byte - 127)` with the low nibble first
(:91-111).  keras int4 kernels: reference tests/test_qmm.py:179-190.
"""
import numpy as np
import pytest

from oracle import qmm_oracle as O
from metaljax_amd import checkpoint as C

E2M1 = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6], np.float32)


def hf_blocks(codes):
    """codes [..., N, K] (0..15) -> HF `_blocks` [..., N, K/32, 16]: byte j of a
    block = element 2j (low nibble) | element 2j+1 (high nibble)."""
    lo, hi = codes[..., 0::2], codes[..., 1::2]
    by = (lo | (hi << 4)).astype(np.uint8)
    return by.reshape(by.shape[:-1] + (by.shape[-1] // 16, 16))


def test_hf_mxfp4_blocks_are_the_kernel_layout_without_a_copy():
    rng = np.random.default_rng(0)
    e, n, k = 2, 5, 128
    codes = rng.integers(0, 16, size=(e, n, k), dtype=np.uint8)
    sb = rng.integers(110, 140, size=(e, n, k // 32)).astype(np.uint8)
    blocks = hf_blocks(codes)
    w, s = C.mxfp4_from_hf_blocks(blocks, sb)
    assert w.shape == (e, n, k // 2) and s.shape == (e, n, k // 32)
    assert np.shares_memory(w, blocks) and s is sb                  # views, not copies
    # the reference's in-graph dequantization, restated
    want = (E2M1[codes].reshape(e, n, k // 32, 32)
            * np.ldexp(np.float32(1), sb.astype(np.int32) - 127)[..., None]).reshape(e, n, k)
    np.testing.assert_array_equal(O.dequant_mxfp4(w, s), want)
    # and the same bytes are the packed uint32 stream (LSB first)
    np.testing.assert_array_equal(np.ascontiguousarray(w).view(np.uint32), O.pack_codes(codes, 4))
    # already-flat codes pass through
    w2, _ = C.mxfp4_from_hf_blocks(w, sb)
    assert w2 is w


@pytest.mark.parametrize("bad", [0, 255])
def test_unusable_e8m0_bytes_are_refused(bad):
    blocks = np.zeros((3, 2, 16), np.uint8)
    sb = np.full((3, 2), 127, np.uint8)
    sb[1, 1] = bad
    with pytest.raises(C.CheckpointFormatError):
        C.mxfp4_from_hf_blocks(blocks, sb)


def test_shapes_and_dtypes_that_do_not_pair_are_refused():
    with pytest.raises(C.CheckpointFormatError):
        C.mxfp4_from_hf_blocks(np.zeros((3, 2, 8), np.uint8), np.full((3, 2), 127, np.uint8))
    with pytest.raises(C.CheckpointFormatError):
        C.mxfp4_from_hf_blocks(np.zeros((3, 4, 16), np.uint8), np.full((3, 2), 127, np.uint8))
    with pytest.raises(C.CheckpointFormatError):
        C.mxfp4_from_hf_blocks(np.zeros((3, 2, 16), np.int8), np.full((3, 2), 127, np.uint8))


def test_safetensors_file_round_trip(tmp_path):
    from safetensors.numpy import save_file
    rng = np.random.default_rng(1)
    codes = rng.integers(0, 16, size=(4, 64), dtype=np.uint8)
    blocks = hf_blocks(codes)
    sb = rng.integers(120, 131, size=(4, 2)).astype(np.uint8)
    path = str(tmp_path / "w.safetensors")
    save_file({"mlp.experts.down_proj_blocks": blocks, "mlp.experts.down_proj_scales": sb}, path)
    w, s = C.load_mxfp4_safetensors(path, "mlp.experts.down_proj_blocks", "mlp.experts.down_proj_scales")
    np.testing.assert_array_equal(np.ascontiguousarray(w).view(np.uint32), O.pack_codes(codes, 4))
    np.testing.assert_array_equal(s, sb)
    with pytest.raises(C.CheckpointFormatError):
        C.load_mxfp4_safetensors(path, "missing_blocks", "mlp.experts.down_proj_scales")


@pytest.mark.parametrize("k,n", [(64, 10), (32, 7)])
def test_keras_int4_kernel_repack(k, n):
    rng = np.random.default_rng(k + n)
    w = rng.integers(-8, 8, size=(k, n)).astype(np.int8)                 # signed int4 [K, N]
    padded = np.concatenate([w, np.zeros((k, n % 2), np.int8)], axis=1)
    packed = ((padded[:, 0::2] & 15) | ((padded[:, 1::2] & 15) << 4)).astype(np.int8)   # keras pack_int4, axis=-1
    np.testing.assert_array_equal(C.keras_int4_unpack(packed, n), w)
    words, offset = C.keras_int4_kernel_to_packed(packed, n)
    assert offset == 8 and words.shape == (n, k // 8) and words.dtype == np.uint32
    np.testing.assert_array_equal(O.unpack_codes(words, 4), (w.T.astype(np.int16) + 8).astype(np.uint8))
    # scale * (q - zero) through pack_exact's offset: biases = -(s * (z + 8))
    s = rng.uniform(0.01, 0.02, (n, k // 32)).astype(np.float32)
    z = rng.integers(-3, 4, (n, k // 32)).astype(np.float32)
    ss, bb, _ = O.scale_bias(s, z, offset, None, "f32")
    got = O.dequant_affine(words, ss, bb, 32, 4)
    want = (w.T.astype(np.float32) - np.repeat(z, 32, axis=1)) * np.repeat(s, 32, axis=1)
    np.testing.assert_allclose(got, want, rtol=0, atol=2e-7)
