"""GPU parity: the HIP path (through the C ABI, via metaljax_amd.kernels)
against the CPU oracle on the same seeded inputs.

Two correctness levels:
  * unpacked codes and dequantized tiles: BIT-EXACT;
  * outputs: rel-L2 <= 1e-2 for bf16 outputs, <= 1e-3 for float32 outputs
    (float32 accumulate).  The decode kernel keeps the weight exact, so it is
    checked against the exactly reconstructed weight; the prefill kernel
    stages a bf16 weight tile, so its 1e-3 level is checked against the
    bf16-rounded weight and its distance to the exact weight is bounded at 3e-3.
"""

import numpy as np
import pytest
import torch

from metaljax_amd import kernels as K
from metaljax_amd import synth
from oracle import c_oracle as C
from oracle import qmm_oracle as O

pytestmark = pytest.mark.gpu

TOL_BF16_OUT = 1e-2
TOL_F32_OUT = 1e-3
DEV = "cuda"


def bf16_dev(bits_u16):
    return torch.from_numpy(np.ascontiguousarray(bits_u16).view(np.int16)).to(DEV).view(torch.bfloat16)


def words_dev(w):
    return torch.from_numpy(np.ascontiguousarray(w).view(np.int32)).to(DEV)


def out_f32(y):
    return y.float().cpu().numpy()


def make_affine(rng, n, k, bits, gs, tab="bf16", lead=()):
    codes = rng.integers(0, 1 << bits, size=lead + (n, k), dtype=np.uint8)
    words = O.pack_codes(codes, bits)
    s = rng.uniform(0.005, 0.02, lead + (n, k // gs)).astype(np.float32)
    if tab == "bf16":
        s = O.round_bf16(s)
        b = O.round_bf16(-(rng.integers(0, 1 << bits, s.shape).astype(np.float32)) * s)
        sd, bd = bf16_dev(O.f32_to_bf16_bits(s)), bf16_dev(O.f32_to_bf16_bits(b))
    elif tab == "f16":
        s = s.astype(np.float16).astype(np.float32)
        b = (-(rng.integers(0, 1 << bits, s.shape).astype(np.float32)) * s).astype(np.float16).astype(np.float32)
        sd = torch.from_numpy(s.astype(np.float16)).to(DEV)
        bd = torch.from_numpy(b.astype(np.float16)).to(DEV)
    else:
        b = (-(rng.uniform(0, 1 << bits, s.shape).astype(np.float32)) * s).astype(np.float32)
        sd, bd = torch.from_numpy(s).to(DEV), torch.from_numpy(b).to(DEV)
    return codes, words, s, b, words_dev(words), sd, bd


def make_mxfp4(rng, n, k, lead=(), lo=118, hi=132):
    codes = rng.integers(0, 16, size=lead + (n, k), dtype=np.uint8)
    codes.reshape(-1, k)[0, :16] = np.arange(16)
    words = O.pack_codes(codes, 4)
    sb = rng.integers(lo, hi, size=lead + (n, k // 32)).astype(np.uint8)
    return codes, words, sb, words_dev(words), torch.from_numpy(sb).to(DEV)


def make_x(rng, m, k):
    x = O.round_bf16(rng.standard_normal((m, k)).astype(np.float32))
    return x, bf16_dev(O.f32_to_bf16_bits(x))


# ------------------------------------------------------------ bit-exact ----

def test_library_reports_loaded():
    from metaljax_amd import _lib
    assert _lib.load().qmm_abi_version() == _lib.ABI_VERSION


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("shape", [(1, 32), (5, 128), (3, 4, 64), (257, 4096)])
def test_unpack_and_pack_codes_bit_exact(bits, shape):
    rng = np.random.default_rng(bits + shape[-1])
    codes = rng.integers(0, 1 << bits, size=shape, dtype=np.uint8)
    words = O.pack_codes(codes, bits)
    got = K.unpack_codes(words_dev(words), bits).cpu().numpy()
    np.testing.assert_array_equal(got, codes)
    packed = K.pack_codes(torch.from_numpy(codes).to(DEV), bits).cpu().numpy().view(np.uint32)
    np.testing.assert_array_equal(packed, words)


def test_pack_layout_hand_computed_words():
    codes = (np.arange(32, dtype=np.uint8) % 16).reshape(1, 32)
    packed = K.pack_codes(torch.from_numpy(codes).to(DEV), 4).cpu().numpy().view(np.uint32)
    np.testing.assert_array_equal(packed[0, :2], np.array([0x76543210, 0xFEDCBA98], np.uint32))


def test_empty_inputs():
    assert K.unpack_codes(torch.zeros((0, 4), dtype=torch.int32, device=DEV), 4).shape == (0, 32)
    x = torch.zeros((0, 64), dtype=torch.bfloat16, device=DEV)
    w = torch.zeros((16, 8), dtype=torch.int32, device=DEV)
    s = torch.ones((16, 1), dtype=torch.bfloat16, device=DEV)
    assert K.quantized_matmul(x, w, s, s, group_size=64, bits=4).shape == (0, 16)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("tab", ["bf16", "f32", "f16"])
def test_dequantize_affine_bit_exact(bits, gs, tab):
    rng = np.random.default_rng(bits * 1000 + gs)
    n, k = 48, 512
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs, tab)
    want = O.dequant_affine(words, s, b, gs, bits)
    got = K.dequantize(wd, sd, bd, group_size=gs, bits=bits).cpu().numpy()
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    got16 = K.dequantize(wd, sd, bd, group_size=gs, bits=bits, out_dtype=torch.bfloat16)
    np.testing.assert_array_equal(got16.view(torch.int16).cpu().numpy().view(np.uint16),
                                  O.f32_to_bf16_bits(want))


@pytest.mark.parametrize("zp_kind", ["zero", "const", "random"])
@pytest.mark.parametrize("scale_kind", ["pow2", "bf16", "f32"])
def test_dequantize_of_pack_exact_matrix(zp_kind, scale_kind):
    """The reference's exactness matrix (tests/test_qmm.py:96-132) through the
    product pack + the device dequantize."""
    from metaljax_amd import packing as P
    bits, gs = 4, 64
    rng = np.random.default_rng(400 + gs)
    n, k = 16, 256
    codes = rng.integers(-8, 8, size=(n, k)).astype(np.int32)
    codes[0, :4] = [-8, 7, 0, -1]
    scale = (rng.random((n, k // gs)).astype(np.float32) + 0.5) * 0.03
    if scale_kind == "pow2":
        scale = np.exp2(rng.integers(-8, 2, size=scale.shape)).astype(np.float32)
    elif scale_kind == "bf16":
        scale = O.round_bf16(scale)
    zp = {"zero": np.zeros((n, k // gs), np.int32), "const": np.full((n, k // gs), 3, np.int32),
          "random": rng.integers(-8, 8, (n, k // gs)).astype(np.int32)}[zp_kind]
    want = scale.repeat(gs, 1) * (codes.astype(np.float32) - zp.repeat(gs, 1).astype(np.float32))
    w, s, b = P.pack_exact(codes, scale, zp, bits)
    got = K.dequantize(words_dev(w), torch.from_numpy(s).to(DEV), torch.from_numpy(b).to(DEV),
                       group_size=gs, bits=bits).cpu().numpy()
    if zp_kind == "zero" or scale_kind in ("pow2", "bf16"):
        np.testing.assert_array_equal(got, want)
    else:
        assert np.abs(got - want).max() / np.abs(want).max() < 1e-5


@pytest.mark.parametrize("shape", [(4, 64), (3, 2, 128), (40, 1024)])
def test_dequantize_mxfp4_bit_exact(shape):
    rng = np.random.default_rng(7 + sum(shape))
    *lead, n, k = shape
    codes, words, sb, wd, sd = make_mxfp4(rng, n, k, tuple(lead), lo=1, hi=255)
    want = O.dequant_mxfp4(O.pack_blocks(codes), sb)
    got = K.dequantize(wd, sd, None, group_size=32, bits=4, mode="mxfp4").cpu().numpy()
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    sb2 = np.clip(sb, 100, 150)
    want2 = O.dequant_mxfp4(O.pack_blocks(codes), sb2)
    got16 = K.dequantize(wd, torch.from_numpy(sb2).to(DEV), None, group_size=32, bits=4,
                         mode="mxfp4", out_dtype=torch.bfloat16).float().cpu().numpy()
    np.testing.assert_array_equal(got16, want2)        # exact in bf16 too


def test_take_k():
    rng = np.random.default_rng(3)
    x, xd = make_x(rng, 5, 256)
    perm = rng.permutation(256).astype(np.int32)
    got = K.take_k(xd, torch.from_numpy(perm).to(DEV)).float().cpu().numpy()
    np.testing.assert_array_equal(got, x[:, perm])


# ------------------------------------------------------- decode (M <= 16) ----

@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("m", [1, 3, 16])
def test_gemv_affine(bits, gs, m):
    rng = np.random.default_rng(bits * 100 + gs + m)
    n, k = 200, 1024                      # N not a multiple of 16
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs)
    x, xd = make_x(rng, m, k)
    want = O.qmm(x, words, s, b, gs, bits)
    y32 = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits, out_dtype=torch.float32))
    assert O.rel_l2(y32, want) <= TOL_F32_OUT, O.rel_l2(y32, want)
    assert O.rel_l2(y32, want) <= 2e-5          # in fact far inside the bar
    y16 = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits))
    assert O.rel_l2(y16, want) <= TOL_BF16_OUT
    np.testing.assert_array_equal(y16, O.round_bf16(y32))     # bf16 out = one RNE of the f32 result


@pytest.mark.parametrize("tab", ["f32", "f16"])
def test_gemv_table_dtypes(tab):
    rng = np.random.default_rng(17)
    n, k, gs, bits = 64, 512, 64, 4
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs, tab)
    x, xd = make_x(rng, 2, k)
    want = O.qmm(x, words, s, b, gs, bits)
    y = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits, out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= 2e-5


@pytest.mark.parametrize("k", [32, 96, 4096])
def test_gemv_k_edge_sizes(k):
    rng = np.random.default_rng(k)
    n, gs, bits = 33, 32, 4
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs)
    x, xd = make_x(rng, 4, k)
    want = O.qmm(x, words, s, b, gs, bits)
    y = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits, out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= 2e-5


@pytest.mark.parametrize("m", [1, 7, 16])
def test_gemv_mxfp4(m):
    rng = np.random.default_rng(40 + m)
    n, k = 72, 2048
    codes, words, sb, wd, sd = make_mxfp4(rng, n, k)
    x, xd = make_x(rng, m, k)
    want = O.qmm(x, words, sb, None, 32, 4, "mxfp4")
    y = out_f32(K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4",
                                   out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= 2e-5, O.rel_l2(y, want)


@pytest.mark.parametrize("m,n,k", [
    (1, 8192, 8192),      # two passes, one row: activations of both passes packed into the operand rows
    (4, 5000, 4096),      # one pass, ragged last tile
    (16, 3000, 4096),     # sixteen rows
    (7, 20000, 4096),     # five tiles a workgroup
    (3, 4100, 12288),     # three passes packed by four rows
    (12, 2048, 8192),     # two passes, activations fetched per pass
    (2, 640, 16384),      # four passes packed by four, fewer workgroups than compute units
    (7, 4096, 8192),      # two passes packed by eight, fourteen live operand rows: whole-line loads through the patches
    (4, 2048, 16384),     # four passes packed by four, sixteen live operand rows
])
def test_decode_mxfp4_big_weights_on_the_loader_wavefront_kernel(m, n, k):
    """MXFP4 decode with K a multiple of 512 and at least eight 256-byte slices:
    the loader-wavefront kernel widens the E2M1 codes with the 32-block's
    power-of-two scale applied in the conversion (exact in bf16)."""
    rng = np.random.default_rng(m * 7 + n + k)
    codes, words, sb, wd, sd = make_mxfp4(rng, n, k)
    x, xd = make_x(rng, m, k)
    want = O.qmm(x, words, sb, None, 32, 4, "mxfp4")
    y32 = out_f32(K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4",
                                     out_dtype=torch.float32))
    assert O.rel_l2(y32, want) <= 2e-5, O.rel_l2(y32, want)
    y16 = out_f32(K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4"))
    np.testing.assert_array_equal(y16, O.round_bf16(y32))


@pytest.mark.parametrize("m,n,k", [
    (1, 5760, 2880),      # gpt-oss gate / up projection: five and a half slices, 90 scale bytes a row
    (2, 2880, 2880),      # its down projection
    (4, 5760, 2880),      # whole-line activation loads, four rows an instruction
    (7, 2880, 2880),      # ... eight rows an instruction
    (16, 5760, 2880),     # staged through the patches
    (16, 2880, 2880),
    (3, 1016, 1088),      # two slices and a piece; the weight's last tile is ragged too
    (9, 520, 3520),       # six slices and seven eighths
    (1, 4104, 4032),      # one 64-code chunk short of eight slices
    (5, 136, 1600),
])
def test_decode_mxfp4_ragged_k_on_the_loader_wavefront_kernel(m, n, k):
    """MXFP4 decode whose K is no whole number of 512-code slices (reference
    scripts/model_bench/mxfp4_gpt_oss.py:90-110: hidden size 2880): the last
    slice's pieces and chunks past K read as zeros, the scale rows (K / 32
    bytes, not dword-aligned one by one) are picked out of the tile's
    contiguous run.  Exact products, float32 accumulate: as the whole-slice form."""
    rng = np.random.default_rng(m * 7 + n + k)
    codes, words, sb, wd, sd = make_mxfp4(rng, n, k, lo=100, hi=150)
    x, xd = make_x(rng, m, k)
    want = O.qmm(x, words, sb, None, 32, 4, "mxfp4")
    y32 = out_f32(K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4",
                                     out_dtype=torch.float32))
    assert O.rel_l2(y32, want) <= 2e-5, O.rel_l2(y32, want)
    y16 = out_f32(K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4"))
    np.testing.assert_array_equal(y16, O.round_bf16(y32))


def test_decode_mxfp4_ragged_k_batched_next_to_non_finite_neighbours():
    """The ragged form reads nothing past K: a batch entry's activations end
    where the next entry's begin, and those are infinite here; scale byte 255
    (NaN) in the neighbouring rows' tables must not leak in either."""
    rng = np.random.default_rng(77)
    e, n, k, m = 3, 264, 2880, 2
    codes, words, sb, wd, sd = make_mxfp4(rng, n, k, lead=(e,))
    x = O.round_bf16(rng.standard_normal((e, m, k)).astype(np.float32))
    xd = bf16_dev(O.f32_to_bf16_bits(x))
    want = [O.qmm(x[z], words[z], sb[z], None, 32, 4, "mxfp4") for z in range(e)]
    # entry 1 becomes poison for its neighbours: infinite activations, NaN scales
    x[1] = np.inf
    xd = bf16_dev(O.f32_to_bf16_bits(x))
    sb2 = sb.copy()
    sb2[1] = 255
    y = out_f32(K.quantized_matmul(xd, wd, torch.from_numpy(sb2).to(DEV), None, group_size=32, bits=4,
                                   mode="mxfp4", out_dtype=torch.float32))
    for z in (0, 2):
        assert np.isfinite(y[z]).all() and O.rel_l2(y[z], want[z]) <= 2e-5


@pytest.mark.parametrize("t,topk,e,n", [(1, 4, 32, 5760), (4, 4, 32, 2880), (16, 4, 32, 5760), (16, 2, 5, 264)])
def test_gather_qmm_grouped_decode_mxfp4_ragged_k(t, topk, e, n):
    """gpt-oss expert projections (32 MXFP4 experts, top-4, K = 2880) as the
    expert-indexed product: pairs sorted by expert, an expert's weight streamed
    once for up to sixteen of its pairs, on the ragged form of the
    loader-wavefront kernel."""
    rng = np.random.default_rng(t * 100 + n)
    k = 2880
    _, words, sb, wd, sd = make_mxfp4(rng, n, k, lead=(e,))
    x, xd = make_x(rng, t, k)
    rhs = np.stack([rng.choice(e, size=topk, replace=False) for _ in range(t)]).reshape(-1).astype(np.int32)
    lhs = np.repeat(np.arange(t, dtype=np.int32), topk)
    want = O.gather_qmm(x[:, None, :], words, sb, None, lhs, rhs, 32, 4, "mxfp4")[:, 0]
    y = out_f32(K.gather_qmm(xd, wd, sd, None, torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV),
                             group_size=32, bits=4, mode="mxfp4", out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= 2e-5, O.rel_l2(y, want)


def test_decode_mxfp4_big_weights_batched_with_extreme_scales():
    rng = np.random.default_rng(404)
    e, n, k, m = 2, 1500, 4096, 3
    codes, words, sb, wd, sd = make_mxfp4(rng, n, k, lead=(e,), lo=100, hi=150)
    x = O.round_bf16(rng.standard_normal((e, m, k)).astype(np.float32))
    xd = bf16_dev(O.f32_to_bf16_bits(x))
    y = out_f32(K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4",
                                   out_dtype=torch.float32))
    for z in range(e):
        want = O.qmm(x[z], words[z], sb[z], None, 32, 4, "mxfp4")
        assert O.rel_l2(y[z], want) <= 2e-5


def test_gemv_batched():
    rng = np.random.default_rng(5)
    bsz, n, k = 3, 48, 256
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64, lead=(bsz,))
    x = O.round_bf16(rng.standard_normal((bsz, 2, k)).astype(np.float32))
    xd = bf16_dev(O.f32_to_bf16_bits(x))
    y = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=64, bits=4, out_dtype=torch.float32))
    for z in range(bsz):
        assert O.rel_l2(y[z], O.qmm(x[z], words[z], s[z], b[z], 64, 4)) <= 2e-5


@pytest.mark.parametrize("bits,gs,m,n,k", [
    (4, 64, 16, 7000, 4096),     # 28 rows a workgroup: two tiles, the second ragged
    (4, 128, 5, 9000, 4096),     # group 128, three tiles a workgroup
    (8, 64, 3, 6001, 4096),      # eight-bit codes: 16 K-slices = two passes, N odd
    (8, 128, 16, 12000, 2048),   # eight-bit codes, one pass
    (4, 64, 2, 5000, 8192),      # two passes of four-bit slices
    (4, 64, 1, 16384, 6144),     # 12 slices: the second pass is half empty
    (8, 64, 7, 12000, 4096),     # eight-bit codes, two passes, three tiles a workgroup
    (4, 128, 16, 9000, 8192),    # two passes, group 128
    (4, 64, 3, 10000, 12288),    # three passes
    (4, 64, 4, 28672, 4096),     # few rows of activations, one pass: 112 rows = seven tiles a workgroup
    (4, 64, 1, 28001, 4096),     # the same with N odd: the last tile ragged, the last workgroup short
    (8, 64, 8, 40000, 2048),     # eight-bit codes in one pass; two rounds of workgroups, five tiles each
    (4, 128, 8, 20000, 4096),    # group 128, five tiles a workgroup
    (4, 64, 8, 4100, 4096),      # one pass, small N: one tile a workgroup, 17 rows -> a ragged second tile
    (4, 64, 3, 2048, 4096),      # fewer workgroups than compute units
    (8, 128, 5, 6144, 2048),     # eight-bit codes, group 128, two tiles a workgroup
    (4, 64, 16, 28672, 4096),    # sixteen rows of activations, wide weight: seven tiles a workgroup, activations fetched directly
    (8, 64, 13, 17000, 2048),    # the same with eight-bit codes and a ragged last tile
    (4, 64, 4, 28672, 8192),     # two passes with directly fetched activations, seven tiles' sums in registers
    (4, 128, 7, 20000, 6144),    # the second pass half empty, five tiles, group 128
    (8, 64, 2, 22016, 4096),     # eight-bit codes, two passes, six tiles
    (4, 64, 16, 30000, 12288),   # sixteen rows, wide weight, three passes, eight tiles (the last ragged)
    (4, 64, 4, 4096, 14336),     # 3.5 passes, four rows: every pass's activations packed into the operand's row blocks of four
    (4, 64, 3, 4100, 12288),     # three passes packed by four (one block unused), ragged second tile
    (4, 128, 8, 8192, 8192),     # two passes packed by eight rows, two tiles a workgroup
    (8, 64, 5, 6144, 4096),      # eight-bit codes, two passes packed by eight
    (4, 64, 1, 5000, 14336),     # one row, 3.5 passes
    (4, 64, 5, 4096, 14336),     # five rows do not pack into four passes: the self-loading kernel
])
def test_decode_big_weights_on_the_loader_wavefront_kernel(bits, gs, m, n, k):
    """Shapes big enough for the decode kernel whose loader wavefronts stream
    the operands through LDS (eight K-slices, more than one tile a workgroup):
    several passes, ragged last tiles, both code widths and group sizes."""
    rng = np.random.default_rng(bits * 1000 + gs + m + n)
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs)
    x, xd = make_x(rng, m, k)
    want = O.qmm(x, words, s, b, gs, bits)
    y32 = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits, out_dtype=torch.float32))
    assert O.rel_l2(y32, want) <= 2e-5, O.rel_l2(y32, want)
    y16 = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits))
    np.testing.assert_array_equal(y16, O.round_bf16(y32))


@pytest.mark.parametrize("bits,gs,m,n,k", [
    (4, 64, 4, 9000, 4096),      # one pass, activations fetched directly
    (4, 128, 1, 4096, 4096),     # group 128, one tile a workgroup
    (8, 64, 16, 5000, 2048),     # eight-bit codes, sixteen rows
    (4, 64, 16, 14336, 4096),    # sixteen rows, 56 rows a workgroup: activations staged through LDS patches
    (4, 64, 6, 14336, 4096),     # six rows: whole-line activation loads through the patches
    (8, 128, 8, 7000, 2048),     # the same with eight-bit codes (half as many bytes a slice)
    (4, 64, 3, 3000, 8192),      # two passes, rows packed
    (4, 64, 7, 3000, 8192),      # two passes, rows packed, more than eight live operand rows (staged through the patches)
    (4, 128, 12, 2048, 12288),   # three passes, one tile a workgroup, activations fetched per pass
])
def test_decode_big_weights_float16_tables(bits, gs, m, n, k):
    """float16 scales and biases (what float16 models carry): the loader-wavefront
    kernel splits an entry into two bf16 terms where it is a matrix operand, so
    the result is as exact as with bf16 tables."""
    rng = np.random.default_rng(bits * 100 + gs + m + n + k)
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs, tab="f16")
    x, xd = make_x(rng, m, k)
    want = O.qmm(x, words, s, b, gs, bits)
    y32 = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits, out_dtype=torch.float32))
    assert O.rel_l2(y32, want) <= 2e-5, O.rel_l2(y32, want)
    y16 = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits))
    np.testing.assert_array_equal(y16, O.round_bf16(y32))


@pytest.mark.parametrize("bits,gs,m,n,k", [
    (4, 64, 4, 9000, 4096),      # groups of 64: eight 4-byte entries a row and slice (two table loads)
    (4, 128, 1, 4096, 4096),     # group 128, one tile a workgroup
    (8, 64, 16, 5000, 2048),     # eight-bit codes, sixteen rows
    (8, 128, 3, 6144, 4096),     # eight-bit codes, group 128, two passes
    (4, 64, 16, 14336, 4096),    # sixteen rows, 56 rows a workgroup: activations through the ring
    (4, 64, 3, 3000, 8192),      # two passes, rows packed
    (4, 128, 12, 2048, 12288),   # three passes, one tile a workgroup, activations fetched per pass
    (4, 64, 2, 28001, 4096),     # seven tiles a workgroup, the last ragged
    (4, 128, 7, 9000, 4096),     # seven rows, group 128: whole-line activation loads through the patches
    (4, 64, 6, 9000, 4096),      # six rows, groups of 64: wide table rows leave no patches, direct fetch
    (4, 128, 4, 4096, 14336),    # 3.5 passes packed by four, group 128: sixteen live operand rows through the patches
    (4, 64, 8, 3000, 8192),      # two passes packed by eight, groups of 64: no patches, direct fetch
])
def test_decode_big_weights_float32_tables(bits, gs, m, n, k):
    """float32 scales and biases (biases that do not fit 16 bits): an entry is
    split into three bf16 terms where it is a matrix operand, so the bias term
    keeps its 24 bits."""
    rng = np.random.default_rng(bits * 100 + gs + m + n + k + 32)
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs, tab="f32")
    x, xd = make_x(rng, m, k)
    want = O.qmm(x, words, s, b, gs, bits)
    y32 = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits, out_dtype=torch.float32))
    assert O.rel_l2(y32, want) <= 2e-5, O.rel_l2(y32, want)
    y16 = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits))
    np.testing.assert_array_equal(y16, O.round_bf16(y32))


def test_decode_big_weights_batched_and_gathered():
    rng = np.random.default_rng(99)
    e, n, k = 3, 9000, 4096
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64, lead=(e,))
    x = O.round_bf16(rng.standard_normal((e, 4, k)).astype(np.float32))
    xd = bf16_dev(O.f32_to_bf16_bits(x))
    y = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=64, bits=4, out_dtype=torch.float32))
    for z in range(e):
        assert O.rel_l2(y[z], O.qmm(x[z], words[z], s[z], b[z], 64, 4)) <= 2e-5
    # a few (token, expert) pairs: one decode product each
    lhs = np.array([2, 0, 1, 1, 3], dtype=np.int32)
    rhs = np.array([1, 2, 0, 2, 1], dtype=np.int32)
    xt = x[0]
    xtd = bf16_dev(O.f32_to_bf16_bits(xt))
    want = O.gather_qmm(xt[:, None, :], words, s, b, lhs, rhs)[:, 0]
    yg = out_f32(K.gather_qmm(xtd, wd, sd, bd, torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV),
                              group_size=64, bits=4, out_dtype=torch.float32))
    assert O.rel_l2(yg, want) <= 2e-5


def test_c1_decode_gemv_full_size():
    wl = synth.make(1)
    x, w, s, b, _ = synth.to_device(wl)
    want = C.qmm(wl.x, wl.w, wl.scales, wl.biases, 64, 4, "affine")
    y = K.quantized_matmul(x, w, s, b, group_size=64, bits=4)
    assert O.rel_l2(out_f32(y), want) <= TOL_BF16_OUT
    y32 = K.quantized_matmul(x, w, s, b, group_size=64, bits=4, out_dtype=torch.float32)
    assert O.rel_l2(out_f32(y32), want) <= 1e-5


@pytest.mark.parametrize("m", [1, 16])
def test_c2_small_batch_full_size(m):
    wl = synth.make(2, M=m)
    x, w, s, b, _ = synth.to_device(wl)
    want = C.qmm(wl.x, wl.w, wl.scales, wl.biases, 64, 4, "affine")
    y32 = K.quantized_matmul(x, w, s, b, group_size=64, bits=4, out_dtype=torch.float32)
    assert O.rel_l2(out_f32(y32), want) <= 1e-5
    y = K.quantized_matmul(x, w, s, b, group_size=64, bits=4)
    assert O.rel_l2(out_f32(y), want) <= TOL_BF16_OUT


# -------------------------------------------------------- prefill (M > 16) ----

@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("m,n,k", [(17, 40, 128), (130, 200, 512), (256, 256, 1024), (64, 128, 96)])
def test_gemm_affine(bits, gs, m, n, k):
    if k % gs:
        pytest.skip("K must be a multiple of the group size")
    rng = np.random.default_rng(bits + gs + m)
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs)
    x, xd = make_x(rng, m, k)
    want_tile = O.qmm(x, words, s, b, gs, bits, weight_rounding="bf16")
    want_exact = O.qmm(x, words, s, b, gs, bits)
    y32 = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits, out_dtype=torch.float32))
    assert O.rel_l2(y32, want_tile) <= 2e-5, O.rel_l2(y32, want_tile)
    assert O.rel_l2(y32, want_exact) <= 3e-3
    y16 = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits))
    assert O.rel_l2(y16, want_exact) <= TOL_BF16_OUT


@pytest.mark.parametrize("tab", ["f32", "f16"])
@pytest.mark.parametrize("gs,bits", [(32, 4), (64, 8), (128, 4)])
@pytest.mark.parametrize("k", [512, 320])
def test_gemm_table_dtypes(tab, gs, bits, k):
    """float32 / float16 scale and bias tables on the prefill kernel: K = 512
    fetches them as 16-byte windows, K = 320 entry by entry."""
    if k % gs:
        pytest.skip("K must be a multiple of the group size")
    rng = np.random.default_rng(gs + bits + k)
    m, n = 40, 136
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs, tab)
    x, xd = make_x(rng, m, k)
    want = O.qmm(x, words, s, b, gs, bits, weight_rounding="bf16")
    y = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits, out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= 2e-5, O.rel_l2(y, want)


def test_grouped_qmm_float32_tables_and_eight_bit_codes():
    rng = np.random.default_rng(23)
    e, n, k = 3, 200, 512
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 8, 64, "f32", lead=(e,))
    sizes = np.array([150, 20, 131])
    ro = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    x, xd = make_x(rng, int(ro[-1]), k)
    want = O.grouped_qmm(x, words, s, b, ro, 64, 8, weight_rounding="bf16")
    y = out_f32(K.grouped_qmm(xd, wd, sd, bd, torch.from_numpy(ro).to(DEV), group_size=64, bits=8,
                              out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= 2e-5, O.rel_l2(y, want)


@pytest.mark.parametrize("m,n,k", [(17, 40, 128), (256, 136, 1024)])
def test_gemm_mxfp4(m, n, k):
    rng = np.random.default_rng(m + n)
    codes, words, sb, wd, sd = make_mxfp4(rng, n, k)
    x, xd = make_x(rng, m, k)
    want = O.qmm(x, words, sb, None, 32, 4, "mxfp4")
    y32 = out_f32(K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4",
                                     out_dtype=torch.float32))
    assert O.rel_l2(y32, want) <= TOL_F32_OUT, O.rel_l2(y32, want)
    y16 = out_f32(K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4"))
    assert O.rel_l2(y16, want) <= TOL_BF16_OUT


@pytest.mark.parametrize("m,n,k", [(70, 200, 512), (64, 128, 2048), (300, 260, 1536), (33, 8, 1024)])
def test_mxfp4_block_scaled_matrix_core_path(m, n, k):
    """K % 512 == 0 and M > 16 runs on the block-scaled matrix cores: the weight
    is exact there, the activations are split into two FP6 terms (about 3e-4
    of |x| left over), so the float32 output must sit within 1e-3 of the oracle."""
    from metaljax_amd import _lib
    import ctypes
    kern = ctypes.c_int()
    assert _lib.load().qmm_plan(m, n, k, 32, 4, 1, kern, None, None) == 0
    assert kern.value == _lib.KERNEL_MXFP4_MFMA
    rng = np.random.default_rng(m * 7 + n)
    codes, words, sb, wd, sd = make_mxfp4(rng, n, k)
    x, xd = make_x(rng, m, k)
    want = O.qmm(x, words, sb, None, 32, 4, "mxfp4")
    y32 = out_f32(K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4",
                                     out_dtype=torch.float32))
    assert O.rel_l2(y32, want) <= TOL_F32_OUT, O.rel_l2(y32, want)
    y16 = out_f32(K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4"))
    assert O.rel_l2(y16, want) <= TOL_BF16_OUT


def test_mxfp4_matrix_core_path_extreme_scales_and_zero_rows():
    """E8M0 bytes over the whole legal range, an all-zero activation row and a
    row of large magnitudes: no NaN/Inf, and the same tolerance row by row."""
    rng = np.random.default_rng(99)
    m, n, k = 40, 96, 512
    codes, words, sb, wd, sd = make_mxfp4(rng, n, k, lo=100, hi=150)
    x, _ = make_x(rng, m, k)
    x[3] = 0.0
    x[5] = O.round_bf16(x[5] * 1.0e4)
    x[7] = O.round_bf16(x[7] * 1.0e-6)
    xd = bf16_dev(O.f32_to_bf16_bits(x))
    want = O.qmm(x, words, sb, None, 32, 4, "mxfp4")
    y = out_f32(K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4",
                                   out_dtype=torch.float32))
    assert np.isfinite(y).all()
    assert not y[3].any()
    for r in (0, 5, 7, 39):
        assert O.rel_l2(y[r], want[r]) <= TOL_F32_OUT, (r, O.rel_l2(y[r], want[r]))


def test_mxfp4_matrix_core_path_batched():
    rng = np.random.default_rng(5)
    bsz, m, n, k = 3, 48, 72, 512
    codes, words, sb, wd, sd = make_mxfp4(rng, n, k, lead=(bsz,))
    x = O.round_bf16(rng.standard_normal((bsz, m, k)).astype(np.float32))
    xd = bf16_dev(O.f32_to_bf16_bits(x))
    y = out_f32(K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4",
                                   out_dtype=torch.float32))
    for z in range(bsz):
        want = O.qmm(x[z], words[z], sb[z], None, 32, 4, "mxfp4")
        assert O.rel_l2(y[z], want) <= TOL_F32_OUT


def test_mxfp4_missing_workspace_is_an_error():
    from metaljax_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(1)
    codes, words, sb, wd, sd = make_mxfp4(rng, 128, 512)
    x, xd = make_x(rng, 64, 512)
    y = torch.empty((64, 128), dtype=torch.bfloat16, device=DEV)
    assert lib.qmm_workspace_bytes(1, 64, 128, 512, 32, 4, 1, _lib.BF16) > 0
    rc = lib.qmm_quantized_matmul(xd.data_ptr(), _lib.BF16, wd.data_ptr(), sd.data_ptr(), None,
                                  _lib.BF16, y.data_ptr(), _lib.BF16, 1, 64, 128, 512, 32, 4, 1,
                                  None, 0, None)
    assert rc == 4 and b"workspace" in lib.qmm_last_error()


def test_c4_mxfp4_scaled_and_full_size():
    wl = synth.make(4, scale=0.125)                      # N = 1024 rows of the same draw
    x, w, s, b, _ = synth.to_device(wl)
    want = C.qmm(wl.x, wl.w, wl.scales, None, 32, 4, "mxfp4", round_tile_bf16=False)
    y32 = K.quantized_matmul(x, w, s, None, group_size=32, bits=4, mode="mxfp4", out_dtype=torch.float32)
    assert O.rel_l2(out_f32(y32), want) <= TOL_F32_OUT, O.rel_l2(out_f32(y32), want)
    # full size: against a float32 torch matmul on the device-dequantized (exact) weight
    wl = synth.make(4)
    x, w, s, b, _ = synth.to_device(wl)
    y = K.quantized_matmul(x, w, s, None, group_size=32, bits=4, mode="mxfp4", out_dtype=torch.float32)
    tile = K.dequantize(w, s, None, group_size=32, bits=4, mode="mxfp4", out_dtype=torch.float32)
    ref = x.float() @ tile.T
    rel = ((y - ref).norm() / ref.norm()).item()
    assert rel <= TOL_F32_OUT, rel
    yb = K.quantized_matmul(x, w, s, None, group_size=32, bits=4, mode="mxfp4")
    assert ((yb.float() - ref).norm() / ref.norm()).item() <= TOL_BF16_OUT


def test_c3_prefill_scaled_and_full_size_properties():
    wl = synth.make(3, scale=0.125, M=256)             # N = 512 rows of the same draw
    x, w, s, b, _ = synth.to_device(wl)
    want = C.qmm(wl.x, wl.w, wl.scales, wl.biases, 64, 8, "affine", round_tile_bf16=True)
    y32 = K.quantized_matmul(x, w, s, b, group_size=64, bits=8, out_dtype=torch.float32)
    assert O.rel_l2(out_f32(y32), want) <= 2e-5
    # full size: against a float32 torch matmul on the device-dequantized bf16 tile
    wl = synth.make(3)
    x, w, s, b, _ = synth.to_device(wl)
    y = K.quantized_matmul(x, w, s, b, group_size=64, bits=8, out_dtype=torch.float32)
    tile = K.dequantize(w, s, b, group_size=64, bits=8, out_dtype=torch.bfloat16)
    ref = x.float() @ tile.float().T
    rel = ((y - ref).norm() / ref.norm()).item()
    assert rel <= 1e-4, rel
    # linearity in x (size-independent property): f(2x) == 2 f(x) exactly in f32
    y2 = K.quantized_matmul(x * 2, w, s, b, group_size=64, bits=8, out_dtype=torch.float32)
    assert torch.equal(y2, y * 2)


@pytest.mark.parametrize("bits,gs,k", [(4, 64, 512), (8, 64, 1024), (4, 128, 768), (4, 32, 256)])
def test_prefill_rows_around_the_borders_of_the_split_role_kernels_tiles(bits, gs, k):
    """Dense products at M > 16 with bf16 tables and K % 256 == 0 run on the
    split-role kernel as one expert of all rows: 256-row tiles dealt as
    contiguous runs, the last tile with 1..256 rows (each of its three loops),
    a ragged last column tile, both epilogues, a batch axis."""
    rng = np.random.default_rng(400 + bits + gs + k)
    n = 264
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs)
    for m in (17, 128, 129, 160, 161, 255, 256, 257, 256 + 140, 600):
        x, xd = make_x(rng, m, k)
        want = O.qmm(x, words, s, b, gs, bits, weight_rounding="bf16")
        y32 = K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits, out_dtype=torch.float32)
        assert O.rel_l2(out_f32(y32), want) <= 2e-5, (m, O.rel_l2(out_f32(y32), want))
        # every row by itself: a row block that went missing would hide in the total
        err = np.abs(out_f32(y32) - want).max(axis=1) / np.abs(want).max()
        assert err.max() <= 1e-4, (m, int(err.argmax()), err.max())
        y16 = K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits)
        assert torch.equal(y16, y32.to(torch.bfloat16)), m
    # two weights at once: the batch axis launches the kernel once per pair
    _, words2, s2, b2, wd2, sd2, bd2 = make_affine(rng, n, k, bits, gs, lead=(2,))
    x = O.round_bf16(rng.standard_normal((2, 300, k)).astype(np.float32))
    xd = bf16_dev(O.f32_to_bf16_bits(x))
    y = out_f32(K.quantized_matmul(xd, wd2, sd2, bd2, group_size=gs, bits=bits, out_dtype=torch.float32))
    for z in range(2):
        want = O.qmm(x[z], words2[z], s2[z], b2[z], gs, bits, weight_rounding="bf16")
        assert O.rel_l2(y[z], want) <= 2e-5, z


@pytest.mark.parametrize("bits,gs,k", [(4, 64, 3584), (4, 64, 3072), (4, 128, 2560), (4, 64, 2048), (8, 64, 1536),
                                       (8, 128, 1024), (4, 64, 1536), (8, 64, 768)])
def test_decode_with_three_to_seven_k_slices_a_row(bits, gs, k):
    """K between three and seven 256-byte slices a row (hidden sizes 1536 to
    3584 with four-bit codes) runs the one-pass loader-wavefront kernel with
    some compute wavefronts idle: every row count's way of fetching the
    activations (direct, whole lines, staged), small and large N (one tile a
    workgroup up to several, and above 64 rows a workgroup also at M > 8), a
    ragged last tile, float16 tables, both outputs, a batch axis."""
    rng = np.random.default_rng(bits * 100 + k)
    for n, ms in ((200, (1, 3, 8, 16)), (5000, (2, 5, 12)), (20011, (1, 4, 7, 9, 16))):
        _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs)
        for m in ms:
            x, xd = make_x(rng, m, k)
            want = O.qmm(x, words, s, b, gs, bits)
            y32 = K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits, out_dtype=torch.float32)
            assert O.rel_l2(out_f32(y32), want) <= 2e-5, (n, m, O.rel_l2(out_f32(y32), want))
            err = np.abs(out_f32(y32) - want).max(axis=0) / np.abs(want).max()      # every output column
            assert err.max() <= 1e-4, (n, m, int(err.argmax()), err.max())
            y16 = K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits)
            assert torch.equal(y16, y32.to(torch.bfloat16)), (n, m)
    # float16 and float32 tables, a batch of two weights, few and many rows of activations
    for tab, m in (("f16", 6), ("f32", 3), ("f16", 13), ("f32", 16)):
        _, words, s, b, wd, sd, bd = make_affine(rng, 3000, k, bits, gs, tab, lead=(2,))
        x = O.round_bf16(rng.standard_normal((2, m, k)).astype(np.float32))
        y = out_f32(K.quantized_matmul(bf16_dev(O.f32_to_bf16_bits(x)), wd, sd, bd, group_size=gs, bits=bits,
                                       out_dtype=torch.float32))
        for z in range(2):
            want = O.qmm(x[z], words[z], s[z], b[z], gs, bits)
            assert O.rel_l2(y[z], want) <= 2e-5, (tab, m, z)


@pytest.mark.parametrize("k", [1536, 2048, 3072, 3584])
def test_mxfp4_decode_with_three_to_seven_k_slices_a_row(k):
    """MXFP4 weights with K between three and seven 512-code slices a row on
    the one-pass loader-wavefront kernel: every row count's way of fetching the
    activations, small and large N, a ragged last tile, both outputs."""
    rng = np.random.default_rng(k)
    for n, ms in ((200, (1, 3, 8, 16)), (5000, (2, 5, 12)), (20011, (1, 4, 9, 16))):
        _, words, sb, wd, sd = make_mxfp4(rng, n, k)
        for m in ms:
            x, xd = make_x(rng, m, k)
            want = O.qmm(x, words, sb, None, 32, 4, "mxfp4")
            y32 = K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4", out_dtype=torch.float32)
            assert O.rel_l2(out_f32(y32), want) <= 2e-5, (n, m, O.rel_l2(out_f32(y32), want))
            err = np.abs(out_f32(y32) - want).max(axis=0) / np.abs(want).max()      # every output column
            assert err.max() <= 1e-4, (n, m, int(err.argmax()), err.max())
            y16 = K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4")
            assert torch.equal(y16, y32.to(torch.bfloat16)), (n, m)


# ----------------------------------------------------------- grouped / MoE ----

def test_grouped_qmm_with_empty_and_ragged_experts():
    rng = np.random.default_rng(21)
    e, n, k = 5, 136, 256
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64, lead=(e,))
    sizes = np.array([3, 0, 130, 1, 0])
    ro = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    x, xd = make_x(rng, int(ro[-1]), k)
    want = O.grouped_qmm(x, words, s, b, ro, 64, 4, weight_rounding="bf16")
    y = out_f32(K.grouped_qmm(xd, wd, sd, bd, torch.from_numpy(ro).to(DEV), group_size=64, bits=4,
                              out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= 2e-5, O.rel_l2(y, want)


@pytest.mark.parametrize("bits,tab", [(4, "bf16"), (8, "bf16"), (4, "f32")])
def test_grouped_qmm_experts_around_one_row_block_past_half_a_tile(bits, tab):
    """256-row tiles: experts of up to 128 rows run one row block a wavefront,
    129..160 rows a fifth block split by columns, more the full tile.  Sizes on
    both sides of each border, both epilogues (float32 and 16-byte bf16 stores),
    a last column tile of 8 columns."""
    rng = np.random.default_rng(77 + bits)
    sizes = np.array([128, 129, 160, 161, 145, 97, 256])
    e, n, k = len(sizes), 264, 512
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, 64, tab, lead=(e,))
    ro = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    x, xd = make_x(rng, int(ro[-1]), k)
    want = O.grouped_qmm(x, words, s, b, ro, 64, bits, weight_rounding="bf16")
    ro_d = torch.from_numpy(ro).to(DEV)
    y32 = out_f32(K.grouped_qmm(xd, wd, sd, bd, ro_d, group_size=64, bits=bits, out_dtype=torch.float32))
    assert O.rel_l2(y32, want) <= 2e-5, O.rel_l2(y32, want)
    y16 = out_f32(K.grouped_qmm(xd, wd, sd, bd, ro_d, group_size=64, bits=bits))
    for i in range(e):                       # every expert's rows by themselves
        lo, hi = ro[i], ro[i + 1]
        assert O.rel_l2(y32[lo:hi], want[lo:hi]) <= 2e-5, (i, O.rel_l2(y32[lo:hi], want[lo:hi]))
        assert O.rel_l2(y16[lo:hi], want[lo:hi]) <= TOL_BF16_OUT, i
    # the 16-bit result is the float32 one rounded once
    assert np.array_equal(y16, out_f32(torch.from_numpy(y32).to(DEV).to(torch.bfloat16)))


@pytest.mark.parametrize("bits,gs,k", [(4, 64, 512), (4, 32, 768), (4, 128, 256), (8, 64, 1024)])
def test_grouped_qmm_short_experts_on_the_split_role_kernel(bits, gs, k):
    """bf16 tables and K % 256 == 0 run the kernel whose wavefronts are split
    into dequantizing producers and multiplying consumers.  Its tiles hold up
    to 256 rows and pick their loop by the rows they hold: up to 128 (one row
    block a consumer), up to 160 (a fifth row block split by columns), more
    (two row blocks a consumer); longer experts in several tiles, an empty
    expert, a last column tile of 8 columns, both epilogues, and the gathered
    form's row scatter."""
    rng = np.random.default_rng(91 + bits + gs)
    sizes = np.array([128, 129, 160, 161, 145, 97, 33, 0, 320, 1, 200, 257, 256])
    e, n = len(sizes), 264
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs, lead=(e,))
    ro = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    r = int(ro[-1])
    x, xd = make_x(rng, r, k)
    want = O.grouped_qmm(x, words, s, b, ro, gs, bits, weight_rounding="bf16")
    ro_d = torch.from_numpy(ro).to(DEV)
    y32 = out_f32(K.grouped_qmm(xd, wd, sd, bd, ro_d, group_size=gs, bits=bits, out_dtype=torch.float32))
    y16 = out_f32(K.grouped_qmm(xd, wd, sd, bd, ro_d, group_size=gs, bits=bits))
    for i in range(e):                       # every expert's rows by themselves
        lo, hi = ro[i], ro[i + 1]
        if hi > lo:
            assert O.rel_l2(y32[lo:hi], want[lo:hi]) <= 2e-5, (i, O.rel_l2(y32[lo:hi], want[lo:hi]))
            assert O.rel_l2(y16[lo:hi], want[lo:hi]) <= TOL_BF16_OUT, i
    # the 16-bit result is the float32 one rounded once
    assert np.array_equal(y16, out_f32(torch.from_numpy(y32).to(DEV).to(torch.bfloat16)))
    # the same products as unsorted (token, expert) pairs
    rhs = np.repeat(np.arange(e), sizes).astype(np.int32)
    perm = rng.permutation(r)
    yg = out_f32(K.gather_qmm(xd, wd, sd, bd, torch.from_numpy(perm.astype(np.int32)).to(DEV),
                              torch.from_numpy(rhs[perm]).to(DEV), group_size=gs, bits=bits,
                              out_dtype=torch.float32))
    assert O.rel_l2(yg, want[perm]) <= 2e-5, O.rel_l2(yg, want[perm])


def test_grouped_qmm_into_a_given_output_leaves_uncovered_rows_alone():
    """out=: rows inside the offsets are written, the others keep what they
    held (a fresh output has zeros there)."""
    rng = np.random.default_rng(33)
    e, n, k = 2, 72, 256
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64, lead=(e,))
    ro = np.array([2, 40, 61], dtype=np.int32)          # rows 0-1 and 61-63 belong to no expert
    x, xd = make_x(rng, 64, k)
    want = O.grouped_qmm(x, words, s, b, ro, 64, 4, weight_rounding="bf16")
    ro_d = torch.from_numpy(ro).to(DEV)
    fresh = out_f32(K.grouped_qmm(xd, wd, sd, bd, ro_d, group_size=64, bits=4, out_dtype=torch.float32))
    assert not fresh[:2].any() and not fresh[61:].any()
    given = torch.full((64, n), 7.0, dtype=torch.float32, device=DEV)
    ret = K.grouped_qmm(xd, wd, sd, bd, ro_d, group_size=64, bits=4, out=given)
    assert ret is given
    got = out_f32(given)
    assert np.array_equal(got[2:61], fresh[2:61])
    assert (got[:2] == 7.0).all() and (got[61:] == 7.0).all()
    assert O.rel_l2(got[2:61], want[2:61]) <= 2e-5
    with pytest.raises(ValueError):
        K.grouped_qmm(xd, wd, sd, bd, ro_d, group_size=64, bits=4, out=given[:, :8])


@pytest.mark.parametrize("pairs", [8, 300])
def test_gather_qmm_unsorted_pairs(pairs):
    """Token-major, unsorted (token, expert) pairs as mx.gather_qmm takes them."""
    rng = np.random.default_rng(pairs)
    e, n, k, t = 4, 64, 256, pairs // 2
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64, lead=(e,))
    x, xd = make_x(rng, t, k)
    lhs = np.repeat(np.arange(t), 2).astype(np.int32)
    rhs = rng.integers(0, e, size=pairs).astype(np.int32)
    rounding = "f32" if pairs <= 64 else "bf16"
    want = O.gather_qmm(x[:, None, :], words, s, b, lhs, rhs, weight_rounding=rounding)[:, 0]
    y = out_f32(K.gather_qmm(xd, wd, sd, bd, torch.from_numpy(lhs).to(DEV),
                             torch.from_numpy(rhs).to(DEV), group_size=64, bits=4,
                             out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= 2e-5, O.rel_l2(y, want)


@pytest.mark.parametrize("bits,mode", [(4, "affine"), (8, "affine"), (4, "mxfp4")])
def test_gather_qmm_many_pairs_skewed_experts(bits, mode):
    """Prefill-sized pair lists: one expert takes most pairs, one takes none,
    and the rows come back in pair order whatever the sort inside did."""
    rng = np.random.default_rng(100 + bits + len(mode))
    e, n, k, t = 6, 200, 512, 700
    if mode == "affine":
        _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, 64, lead=(e,))
        gs = 64
    else:
        _, words, s, wd, sd = make_mxfp4(rng, n, k, lead=(e,))
        b, bd, gs = None, None, 32
    x, xd = make_x(rng, t, k)
    p = 2 * t
    lhs = rng.permutation(np.repeat(np.arange(t), 2)).astype(np.int32)
    rhs = rng.choice(e, size=p, p=[0.7, 0.1, 0.0, 0.1, 0.05, 0.05]).astype(np.int32)
    want = O.gather_qmm(x[:, None, :], words, s, b, lhs, rhs, gs, bits, mode,
                        weight_rounding="bf16")[:, 0]
    y = out_f32(K.gather_qmm(xd, wd, sd, bd, torch.from_numpy(lhs).to(DEV),
                             torch.from_numpy(rhs).to(DEV), group_size=gs, bits=bits, mode=mode,
                             out_dtype=torch.float32))
    # MXFP4 at K % 512 == 0 runs on the block-scaled matrix cores (two FP6 activation terms)
    tol = TOL_F32_OUT if mode == "mxfp4" else 2e-5
    assert O.rel_l2(y, want) <= tol, O.rel_l2(y, want)
    # bf16 results, identity lhs (pair p reads row p)
    want2 = O.gather_qmm(x[:, None, :], words, s, b, np.arange(t), rhs[:t], gs, bits, mode,
                         weight_rounding="bf16")[:, 0]
    y2 = out_f32(K.gather_qmm(xd, wd, sd, bd, None, torch.from_numpy(rhs[:t]).to(DEV),
                              group_size=gs, bits=bits, mode=mode))
    assert O.rel_l2(y2, want2) <= 1e-2, O.rel_l2(y2, want2)


def test_gather_qmm_pairs_naming_no_expert_are_skipped():
    """An expert index outside [0, E) selects nothing: the pair's row is left
    as it was and every other row is right."""
    rng = np.random.default_rng(77)
    e, n, k, t = 3, 72, 256, 90
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64, lead=(e,))
    x, xd = make_x(rng, t, k)
    lhs = np.arange(t).astype(np.int32)
    rhs = rng.integers(0, e, size=t).astype(np.int32)
    bad = np.array([4, 17, 60])
    rhs_dev = rhs.copy()
    rhs_dev[bad] = [e, -1, 1000]
    want = O.gather_qmm(x[:, None, :], words, s, b, lhs, rhs, weight_rounding="bf16")[:, 0]
    y = out_f32(K.gather_qmm(xd, wd, sd, bd, torch.from_numpy(lhs).to(DEV),
                             torch.from_numpy(rhs_dev).to(DEV), group_size=64, bits=4,
                             out_dtype=torch.float32))
    good = np.setdiff1d(np.arange(t), bad)
    assert O.rel_l2(y[good], want[good]) <= 2e-5


def test_gather_qmm_with_only_the_sort_workspace_still_runs():
    """The C entry point accepts the smaller workspace (the expert sort's arrays
    alone) and serves the call on the general kernel."""
    from metaljax_amd import _lib
    from metaljax_amd.kernels import _ptr, _dt, _stream
    lib = _lib.load()
    rng = np.random.default_rng(5)
    e, n, k, t = 4, 64, 256, 150
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64, lead=(e,))
    x, xd = make_x(rng, t, k)
    rhs = rng.integers(0, e, size=t).astype(np.int32)
    rd = torch.from_numpy(rhs).to(DEV)
    full = int(lib.qmm_gather_workspace_bytes(t, e, n, k, _lib.BF16))
    small = ((2 * e + 1 + 2 * t) * 4 + 255) // 256 * 256
    assert full > small
    ws = torch.empty(small, dtype=torch.uint8, device=DEV)
    y = torch.empty((t, n), dtype=torch.float32, device=DEV)
    rc = lib.qmm_gather_qmm(_ptr(xd), _lib.BF16, _ptr(wd), _ptr(sd), _ptr(bd), _lib.BF16, _ptr(y),
                            _dt(torch.float32), None, _ptr(rd), t, t, e, n, k, 64, 4, 0, _ptr(ws),
                            small, _stream(xd))
    assert rc == 0, lib.qmm_last_error()
    want = O.gather_qmm(x[:, None, :], words, s, b, np.arange(t), rhs, weight_rounding="bf16")[:, 0]
    assert O.rel_l2(out_f32(y), want) <= 2e-5
    rc = lib.qmm_gather_qmm(_ptr(xd), _lib.BF16, _ptr(wd), _ptr(sd), _ptr(bd), _lib.BF16, _ptr(y),
                            _dt(torch.float32), None, _ptr(rd), t, t, e, n, k, 64, 4, 0, _ptr(ws),
                            small - 256, _stream(xd))
    assert rc == 4 and _lib.ERR_NAMES[rc] == "WORKSPACE"


@pytest.mark.parametrize("k", [1024, 768])
def test_grouped_and_gathered_mxfp4_experts(k):
    """MXFP4 experts (the gpt-oss layout): K % 512 == 0 runs the expert products
    on the block-scaled matrix cores (tiles never straddle an expert, empty and
    ragged experts, rows gathered and scattered), other K on the bf16 kernel."""
    rng = np.random.default_rng(k)
    e, n = 5, 200
    _, words, sb, wd, sd = make_mxfp4(rng, n, k, lead=(e,))
    sizes = np.array([70, 0, 129, 3, 64])
    ro = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    r = int(ro[-1])
    x, xd = make_x(rng, r, k)
    want = O.grouped_qmm(x, words, sb, None, ro, 32, 4, "mxfp4")
    tol = TOL_F32_OUT if k % 512 == 0 else 2e-5
    y = out_f32(K.grouped_qmm(xd, wd, sd, None, torch.from_numpy(ro).to(DEV), group_size=32, bits=4,
                              mode="mxfp4", out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= tol, O.rel_l2(y, want)
    for a, b in zip(ro[:-1], ro[1:]):                       # every expert's rows on their own
        if b > a:
            assert O.rel_l2(y[a:b], want[a:b]) <= tol
    y16 = out_f32(K.grouped_qmm(xd, wd, sd, None, torch.from_numpy(ro).to(DEV), group_size=32, bits=4,
                                mode="mxfp4"))
    assert O.rel_l2(y16, want) <= TOL_BF16_OUT
    rhs = np.repeat(np.arange(e), sizes).astype(np.int32)
    perm = rng.permutation(r)
    yg = out_f32(K.gather_qmm(xd, wd, sd, None, torch.from_numpy(perm.astype(np.int32)).to(DEV),
                              torch.from_numpy(rhs[perm]).to(DEV), group_size=32, bits=4, mode="mxfp4",
                              out_dtype=torch.float32))
    assert O.rel_l2(yg, want[perm]) <= tol, O.rel_l2(yg, want[perm])


@pytest.mark.parametrize("kind", ["bf16 tables", "f32 tables", "mxfp4"])
def test_grouped_qmm_over_many_experts(kind):
    """More experts than a wavefront has lanes (the kernels find a tile's
    expert 64 experts at a time): 150 experts, most with a few rows, some
    empty, some longer than one row tile of any kernel, the last one not
    empty; each of the three grouped prefill kernels; the gathered form."""
    rng = np.random.default_rng(len(kind))
    e, n, k = 150, 136, 512
    sizes = rng.integers(0, 6, size=e)
    sizes[rng.choice(e, size=20, replace=False)] = 0
    sizes[[3, 70, 149]] = [300, 170, 7]
    ro = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    r = int(ro[-1])
    x, xd = make_x(rng, r, k)
    ro_d = torch.from_numpy(ro).to(DEV)
    if kind == "mxfp4":
        _, words, s, wd, sd = make_mxfp4(rng, n, k, lead=(e,))
        b, bd, gs, mode, rounding, tol = None, None, 32, "mxfp4", "f32", TOL_F32_OUT
    else:
        _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64, "bf16" if kind == "bf16 tables" else "f32",
                                                 lead=(e,))
        gs, mode, rounding, tol = 64, "affine", "bf16", 2e-5
    want = O.grouped_qmm(x, words, s, b, ro, gs, 4, mode, weight_rounding=rounding)
    y = out_f32(K.grouped_qmm(xd, wd, sd, bd, ro_d, group_size=gs, bits=4, mode=mode, out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= tol, O.rel_l2(y, want)
    for i in range(e):                       # every expert's rows by themselves
        lo, hi = ro[i], ro[i + 1]
        if hi > lo:
            assert O.rel_l2(y[lo:hi], want[lo:hi]) <= 10 * tol, (i, O.rel_l2(y[lo:hi], want[lo:hi]))
    rhs = np.repeat(np.arange(e), sizes).astype(np.int32)
    perm = rng.permutation(r)
    yg = out_f32(K.gather_qmm(xd, wd, sd, bd, torch.from_numpy(perm.astype(np.int32)).to(DEV),
                              torch.from_numpy(rhs[perm]).to(DEV), group_size=gs, bits=4, mode=mode,
                              out_dtype=torch.float32))
    assert O.rel_l2(yg, want[perm]) <= tol, O.rel_l2(yg, want[perm])
    if kind == "bf16 tables":
        # without a workspace the C entry point serves the call on the kernel that stages both operands in LDS
        from metaljax_amd import _lib
        lib = _lib.load()
        y0 = torch.zeros((r, n), dtype=torch.float32, device=DEV)
        rc = lib.qmm_grouped_qmm(xd.data_ptr(), _lib.BF16, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), _lib.BF16,
                                 y0.data_ptr(), _lib.F32, ro_d.data_ptr(), r, e, n, k, gs, 4, 0, None, 0,
                                 torch.cuda.current_stream().cuda_stream)
        assert rc == 0, lib.qmm_last_error()
        assert O.rel_l2(out_f32(y0), want) <= tol, O.rel_l2(out_f32(y0), want)


def test_c5_moe_scaled():
    wl = synth.make(5, scale=1 / 56)                  # N = 256, 18 tokens... of the same draw
    x, w, s, b, ro = synth.to_device(wl)
    want = C.grouped_qmm(wl.x, wl.w, wl.scales, wl.biases, wl.row_offsets, 64, 4, "affine",
                         round_tile_bf16=True)
    y = K.grouped_qmm(x, w, s, b, ro, group_size=64, bits=4, out_dtype=torch.float32)
    assert O.rel_l2(out_f32(y), want) <= 2e-5


# ------------------------------------------------- checkpoint-side layouts ----

def test_hf_mxfp4_checkpoint_tensors_feed_the_kernels_as_they_are():
    """`_blocks` [E, N, K/32, 16] / `_scales` [E, N, K/32] uint8 straight from a
    checkpoint (reference scripts/model_bench/mxfp4_gpt_oss.py:211-258): the
    flattened blocks are the packed weight, no repack on either side."""
    from metaljax_amd import checkpoint as CK
    rng = np.random.default_rng(31)
    e, n, k = 3, 96, 1024
    codes = rng.integers(0, 16, size=(e, n, k), dtype=np.uint8)
    blocks = (codes[..., 0::2] | (codes[..., 1::2] << 4)).astype(np.uint8).reshape(e, n, k // 32, 16)
    sb = rng.integers(118, 132, size=(e, n, k // 32)).astype(np.uint8)
    w, sc = CK.mxfp4_from_hf_blocks(torch.from_numpy(blocks).to(DEV), torch.from_numpy(sb).to(DEV))
    assert tuple(w.shape) == (e, n, k // 2) and sc.dtype == torch.uint8
    x, xd = make_x(rng, 40, k)
    words = O.pack_codes(codes, 4)
    # one expert as a plain product (prefill and decode), all of them as a gathered product
    want = O.qmm(x, words[1], sb[1], None, 32, 4, "mxfp4")
    y = out_f32(K.quantized_matmul(xd, w[1], sc[1], None, group_size=32, bits=4, mode="mxfp4",
                                   out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= TOL_F32_OUT
    y1 = out_f32(K.quantized_matmul(xd[:2], w[1], sc[1], None, group_size=32, bits=4, mode="mxfp4",
                                    out_dtype=torch.float32))
    assert O.rel_l2(y1, want[:2]) <= 2e-5
    rhs = rng.integers(0, e, size=40).astype(np.int32)
    wantg = O.gather_qmm(x[:, None, :], words, sb, None, np.arange(40), rhs, 32, 4, "mxfp4")[:, 0]
    yg = out_f32(K.gather_qmm(xd, w, sc, None, None, torch.from_numpy(rhs).to(DEV), group_size=32, bits=4,
                              mode="mxfp4", out_dtype=torch.float32))
    assert O.rel_l2(yg, wantg) <= TOL_F32_OUT


def test_keras_int4_kernel_repacked_once_then_multiplied():
    from metaljax_amd import checkpoint as CK
    rng = np.random.default_rng(32)
    k, n = 512, 72
    wq = rng.integers(-8, 8, size=(k, n)).astype(np.int8)
    packed = ((wq[:, 0::2] & 15) | ((wq[:, 1::2] & 15) << 4)).astype(np.int8)
    words, offset = CK.keras_int4_kernel_to_packed(packed, n)
    s = O.round_bf16(rng.uniform(0.005, 0.02, (n, k // 64)).astype(np.float32))
    z = rng.integers(-2, 3, (n, k // 64)).astype(np.float32)
    ss, bb, kind = O.scale_bias(s, z, offset, "bf16")
    x, xd = make_x(rng, 3, k)
    want = x @ ((wq.T.astype(np.float32) - np.repeat(z, 64, axis=1)) * np.repeat(s, 64, axis=1)).T
    tab = (lambda v: bf16_dev(O.f32_to_bf16_bits(v))) if kind == "bf16" else (lambda v: torch.from_numpy(v).to(DEV))
    y = out_f32(K.quantized_matmul(xd, CK.to_device(words), tab(ss), tab(bb), group_size=64, bits=4,
                                   out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= 2e-5, O.rel_l2(y, want)


# ------------------------------------------------------------ error paths ----

def test_unsupported_and_bad_shapes_raise_without_launching():
    x = torch.zeros((2, 64), dtype=torch.bfloat16, device=DEV)
    w = torch.zeros((16, 8), dtype=torch.int32, device=DEV)
    s = torch.ones((16, 1), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(K.UnsupportedQmm):
        K.quantized_matmul(x, w, s, s, group_size=16, bits=4)
    with pytest.raises(K.UnsupportedQmm):
        K.quantized_matmul(x.double(), w, s, s, group_size=64, bits=4)     # float64 activations
    with pytest.raises(K.QmmError):
        K.quantized_matmul(x, w, s, None, group_size=64, bits=4)       # affine without biases
    with pytest.raises(K.QmmError):
        K.quantized_matmul(x.cpu(), w, s, s, group_size=64, bits=4)    # no CPU path


@pytest.mark.parametrize("bits,gs,t,pairs,e,n,k,skew", [
    (4, 64, 4, 8, 8, 9000, 4096, False),       # top-2 of eight experts for four tokens
    (4, 64, 16, 32, 4, 5000, 4096, False),     # eight pairs an expert on average
    (4, 128, 24, 48, 3, 2100, 4096, True),     # most pairs on one expert: more than sixteen rows = several chunks
    (8, 64, 6, 12, 5, 3000, 2048, False),      # eight-bit codes
    (4, 64, 5, 10, 4, 4100, 8192, False),      # two passes over K (rows packed by eight or fetched per pass)
    (4, 64, 30, 60, 2, 1000, 12288, True),     # three passes, up to sixteen rows an expert chunk
    (4, 64, 50, 100, 8, 3000, 4096, False),    # more than 64 pairs, still at most 16 an expert on average
    (4, 64, 40, 120, 8, 2100, 4096, True),     # most of 120 pairs on one expert: seven of its chunks, a few others
])
def test_gather_qmm_few_pairs_grouped_by_expert(bits, gs, t, pairs, e, n, k, skew):
    """Between 4 and 16 x E pairs: the pairs are sorted by expert and each expert's
    weight is streamed once against its (up to sixteen at a time) rows; results
    come back in pair order."""
    rng = np.random.default_rng(pairs * 31 + e)
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs, lead=(e,))
    x, xd = make_x(rng, t, k)
    lhs = rng.integers(0, t, size=pairs).astype(np.int32)
    rhs = rng.integers(0, e, size=pairs).astype(np.int32)
    if skew:
        rhs[rng.random(pairs) < 0.8] = e - 1
    want = O.gather_qmm(x[:, None, :], words, s, b, lhs, rhs, gs, bits)[:, 0]
    y = out_f32(K.gather_qmm(xd, wd, sd, bd, torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV),
                             group_size=gs, bits=bits, out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= 2e-5, O.rel_l2(y, want)
    y16 = out_f32(K.gather_qmm(xd, wd, sd, bd, torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV),
                               group_size=gs, bits=bits))
    np.testing.assert_array_equal(y16, O.round_bf16(y))


def test_gather_qmm_few_pairs_grouped_by_expert_float16_tables():
    rng = np.random.default_rng(1616)
    e, n, k, t, pairs = 4, 2500, 4096, 9, 24
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64, tab="f16", lead=(e,))
    x, xd = make_x(rng, t, k)
    lhs = rng.integers(0, t, size=pairs).astype(np.int32)
    rhs = rng.integers(0, e, size=pairs).astype(np.int32)
    want = O.gather_qmm(x[:, None, :], words, s, b, lhs, rhs, 64, 4)[:, 0]
    y = out_f32(K.gather_qmm(xd, wd, sd, bd, torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV),
                             group_size=64, bits=4, out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= 2e-5, O.rel_l2(y, want)


@pytest.mark.parametrize("gs", [64, 128])
def test_gather_qmm_few_pairs_grouped_by_expert_float32_tables(gs):
    rng = np.random.default_rng(3232 + gs)
    e, n, k, t, pairs = 4, 2500, 4096, 9, 24
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, gs, tab="f32", lead=(e,))
    x, xd = make_x(rng, t, k)
    lhs = rng.integers(0, t, size=pairs).astype(np.int32)
    rhs = rng.integers(0, e, size=pairs).astype(np.int32)
    want = O.gather_qmm(x[:, None, :], words, s, b, lhs, rhs, gs, 4)[:, 0]
    y = out_f32(K.gather_qmm(xd, wd, sd, bd, torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV),
                             group_size=gs, bits=4, out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= 2e-5, O.rel_l2(y, want)


@pytest.mark.parametrize("kind,bits,gs,tab,t,pairs,e,n,k,skew", [
    ("mxfp4", 4, 32, "bf16", 16, 64, 8, 700, 2880, False),      # the gpt-oss width: 5.6 slices, 90 scale bytes a row
    ("mxfp4", 4, 32, "bf16", 9, 40, 3, 300, 1120, True),        # most pairs on one expert: several chunks of sixteen
    ("affine", 4, 64, "bf16", 12, 48, 5, 520, 1088, False),     # K not a whole number of 256-byte slices
    ("affine", 8, 32, "f16", 7, 16, 6, 200, 736, False),        # sixteen pairs: the smallest grouped launch
    ("affine", 4, 128, "f32", 20, 64, 4, 333, 2176, True),
])
def test_gather_qmm_few_pairs_on_the_general_decode_kernels(kind, bits, gs, tab, t, pairs, e, n, k, skew):
    """Sixteen to 64 pairs on shapes that no staged decode kernel serves: the
    pairs are sorted by expert and the general decode kernels multiply up to
    sixteen rows of one expert at a time; a pair naming no expert keeps its
    output row, a pair naming a row outside x multiplies zeros."""
    from metaljax_amd import _lib
    rng = np.random.default_rng(pairs * 7 + k)
    if kind == "mxfp4":
        _, words, s, wd, sd = make_mxfp4(rng, n, k, lead=(e,))
        b, bd = None, None
    else:
        _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs, tab, lead=(e,))
    x, xd = make_x(rng, t, k)
    lhs = rng.integers(0, t, size=pairs).astype(np.int32)
    rhs = rng.integers(0, e, size=pairs).astype(np.int32)
    if skew:
        rhs[rng.random(pairs) < 0.8] = e - 1
    lhs[3], rhs[5], rhs[11] = t + 2, e, -1                 # a row outside x, two pairs naming no expert
    lib = _lib.load()
    nbytes = int(lib.qmm_gather_workspace_bytes(pairs, e, n, k, _lib.BF16))
    assert nbytes > 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    ld, rd = torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV)
    tabd = {"bf16": _lib.BF16, "f16": _lib.F16, "f32": _lib.F32}[tab]
    for yd, ydt in ((_lib.F32, torch.float32), (_lib.BF16, torch.bfloat16)):
        y = torch.full((pairs, n), 7.0, dtype=ydt, device=DEV)
        rc = lib.qmm_gather_qmm(xd.data_ptr(), _lib.BF16, wd.data_ptr(), sd.data_ptr(),
                                None if bd is None else bd.data_ptr(), tabd, y.data_ptr(), yd,
                                ld.data_ptr(), rd.data_ptr(), pairs, t, e, n, k, gs, bits,
                                1 if kind == "mxfp4" else 0, ws.data_ptr(), nbytes,
                                torch.cuda.current_stream().cuda_stream)
        _lib.check(rc)
        got = out_f32(y)
        tol = 2e-5 if yd == _lib.F32 else TOL_BF16_OUT
        for i in range(pairs):
            if not 0 <= rhs[i] < e:
                np.testing.assert_array_equal(got[i], np.full(n, 7.0, np.float32))
            elif not 0 <= lhs[i] < t:
                np.testing.assert_array_equal(got[i], np.zeros(n, np.float32))
            else:
                want = O.qmm(x[lhs[i]][None], words[rhs[i]], s[rhs[i]], None if b is None else b[rhs[i]],
                             gs, bits, kind)[0]
                assert O.rel_l2(got[i], want) <= tol, (i, O.rel_l2(got[i], want))


def test_gather_qmm_few_pairs_invalid_indices_touch_nothing():
    """Grouped decode: a pair naming no expert keeps its output row as it was,
    a pair naming a row outside x multiplies zeros."""
    rng = np.random.default_rng(77)
    e, n, k, t = 4, 2048, 4096, 6
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64, lead=(e,))
    x, xd = make_x(rng, t, k)
    lhs = np.array([0, 5, 2, 9, 1, 3, -1, 4], dtype=np.int32)      # 9 and -1 are outside x
    rhs = np.array([1, 7, 0, 2, -3, 3, 1, 1], dtype=np.int32)      # 7 and -3 name no expert
    from metaljax_amd import _lib
    lib = _lib.load()
    p = len(lhs)
    nbytes = int(lib.qmm_gather_workspace_bytes(p, e, n, k, _lib.BF16))
    assert nbytes > 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    y = torch.full((p, n), 7.0, dtype=torch.float32, device=DEV)
    ld, rd = torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV)
    rc = lib.qmm_gather_qmm(xd.data_ptr(), _lib.BF16, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), _lib.BF16,
                            y.data_ptr(), _lib.F32, ld.data_ptr(), rd.data_ptr(), p, t, e, n, k, 64, 4, 0,
                            ws.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream)
    _lib.check(rc)
    got = y.cpu().numpy()
    for i in range(p):
        if not 0 <= rhs[i] < e:
            np.testing.assert_array_equal(got[i], np.full(n, 7.0, np.float32))
        elif not 0 <= lhs[i] < t:
            np.testing.assert_array_equal(got[i], np.zeros(n, np.float32))
        else:
            want = O.qmm(x[lhs[i]][None], words[rhs[i]], s[rhs[i]], b[rhs[i]], 64, 4)[0]
            assert O.rel_l2(got[i], want) <= 2e-5


@pytest.mark.parametrize("k,pairs,e", [(4096, 20, 6), (8192, 40, 3)])
def test_gather_qmm_few_pairs_grouped_by_expert_mxfp4(k, pairs, e):
    """MXFP4 experts, few pairs: grouped decode on the loader-wavefront kernel."""
    rng = np.random.default_rng(k + pairs)
    n, t = 1200, 10
    _, words, sb, wd, sd = make_mxfp4(rng, n, k, lead=(e,))
    x, xd = make_x(rng, t, k)
    lhs = rng.integers(0, t, size=pairs).astype(np.int32)
    rhs = rng.integers(0, e, size=pairs).astype(np.int32)
    want = O.gather_qmm(x[:, None, :], words, sb, None, lhs, rhs, 32, 4, "mxfp4")[:, 0]
    y = out_f32(K.gather_qmm(xd, wd, sd, None, torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV),
                             group_size=32, bits=4, mode="mxfp4", out_dtype=torch.float32))
    assert O.rel_l2(y, want) <= 2e-5, O.rel_l2(y, want)


@pytest.mark.parametrize("pairs,n,k,mode", [
    (3, 2048, 4096, "affine"),      # below four pairs: independent products on the loader-wavefront kernel
    (32, 2048, 4096, "affine"),     # no workspace: the same, 32 launches' worth of pairs
    (32, 300, 1024, "affine"),      # two K-slices: the self-loading kernel
    (32, 72, 96, "affine"),         # the general decode kernel
    (32, 72, 256, "mxfp4"),         # the general MXFP4 decode kernel
])
def test_gather_qmm_independent_decode_products_check_their_indices(pairs, n, k, mode):
    """Pairs that run as independent decode products (no expert sort): an
    expert index outside [0, E) leaves the pair's output row as it was, a row
    index outside [0, T) multiplies zeros -- what the sorted paths do."""
    from metaljax_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(pairs + n + k)
    e, t = 4, 6
    if mode == "affine":
        _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 32 if k == 96 else 64, lead=(e,))
        gs = 32 if k == 96 else 64
    else:
        _, words, s, wd, sd = make_mxfp4(rng, n, k, lead=(e,))
        b, bd, gs = None, None, 32
    x, xd = make_x(rng, t, k)
    lhs = rng.integers(0, t, size=pairs).astype(np.int32)
    rhs = rng.integers(0, e, size=pairs).astype(np.int32)
    lhs[1] = t                   # one past the last row
    if pairs > 3:
        lhs[7], rhs[5], rhs[9] = -1, e, -2
    else:
        rhs[2] = e + 5
    y = torch.full((pairs, n), 7.0, dtype=torch.float32, device=DEV)
    ld, rd = torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV)
    rc = lib.qmm_gather_qmm(xd.data_ptr(), _lib.BF16, wd.data_ptr(), sd.data_ptr(),
                            None if bd is None else bd.data_ptr(), _lib.BF16, y.data_ptr(), _lib.F32,
                            ld.data_ptr(), rd.data_ptr(), pairs, t, e, n, k, gs, 4,
                            0 if mode == "affine" else 1, None, 0,
                            torch.cuda.current_stream().cuda_stream)
    _lib.check(rc)
    got = y.cpu().numpy()
    for i in range(pairs):
        if not 0 <= rhs[i] < e:
            np.testing.assert_array_equal(got[i], np.full(n, 7.0, np.float32))
        elif not 0 <= lhs[i] < t:
            np.testing.assert_array_equal(got[i], np.zeros(n, np.float32))
        else:
            bi = None if b is None else b[rhs[i]]
            want = O.qmm(x[lhs[i]][None], words[rhs[i]], s[rhs[i]], bi, gs, 4, mode)[0]
            assert O.rel_l2(got[i], want) <= 2e-5, i


@pytest.mark.parametrize("xdt", ["f32", "f16"])
def test_gather_qmm_wide_activations_without_lhs_read_zeros_past_x(xdt):
    """float16 / float32 activations, no lhs indices, more pairs than rows of
    x: pair p reads row p, and the pairs past the last row multiply zeros (the
    split into bf16 terms must not read beyond x), as on the bf16 path."""
    from metaljax_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(77)
    e, t, pairs, n, k = 3, 4, 9, 128, 512
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64, lead=(e,))
    x = rng.standard_normal((t, k)).astype(np.float32)
    if xdt == "f16":
        x = x.astype(np.float16).astype(np.float32)
        xd, code = torch.from_numpy(x).to(DEV).half(), _lib.F16
    else:
        xd, code = torch.from_numpy(x).to(DEV), _lib.F32
    rhs = rng.integers(0, e, size=pairs).astype(np.int32)
    rd = torch.from_numpy(rhs).to(DEV)
    y = torch.full((pairs, n), 7.0, dtype=torch.float32, device=DEV)
    nbytes = int(lib.qmm_gather_workspace_bytes(pairs, e, n, k, code))
    ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    rc = lib.qmm_gather_qmm(xd.data_ptr(), code, wd.data_ptr(), sd.data_ptr(), bd.data_ptr(), _lib.BF16,
                            y.data_ptr(), _lib.F32, None, rd.data_ptr(), pairs, t, e, n, k, 64, 4, 0,
                            ws.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream)
    _lib.check(rc)
    got = y.cpu().numpy()
    for i in range(pairs):
        if i >= t:
            np.testing.assert_array_equal(got[i], np.zeros(n, np.float32))
        else:
            want = O.qmm(x[i][None], words[rhs[i]], s[rhs[i]], b[rhs[i]], 64, 4, "affine")[0]
            assert O.rel_l2(got[i], want) <= 2e-5, i


def test_wide_activations_non_finite_rows_stay_non_finite():
    """A float32 activation row holding inf or NaN gives a non-finite output
    row (the split into bf16 terms keeps inf / NaN in the first term and cuts
    no NaN payload down to inf), and leaves the other rows alone."""
    rng = np.random.default_rng(5)
    n, k = 64, 512
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64)
    x = rng.standard_normal((4, k)).astype(np.float32)
    x[0, 3] = np.inf
    x[1, 5] = np.nan
    x[3, 7] = np.uint32(0x7F800001).view(np.float32)        # a NaN whose payload sits in the low mantissa bits
    y = K.quantized_matmul(torch.from_numpy(x).to(DEV), wd, sd, bd, group_size=64, bits=4,
                           out_dtype=torch.float32).cpu().numpy()
    assert not np.isfinite(y[0]).any()
    assert np.isnan(y[1]).all() and np.isnan(y[3]).all()
    want = O.qmm(x[2][None], words, s, b, 64, 4)[0]
    assert O.rel_l2(y[2], want) <= 2e-5


# ------------------------------------- the named configurations at full size ----

def _report(name, **figures):
    """Measured distances of a full-size configuration, shown with `pytest -s`
    / in the captured output of a failure, and kept for the session summary."""
    line = name + ": " + ", ".join(f"{k} = {v:.3e}" for k, v in figures.items())
    print(line)
    FULL_SIZE_REPORT.append(line)


FULL_SIZE_REPORT = []


def test_c3_prefill_full_size_against_the_oracle():
    """C3 whole (x [2048, 4096] x int8 g64 [4096, 4096]) against the C oracle:
    float32 output against the bf16-rounded weight tile (the tile the kernel
    stages is that rounding, so only accumulation order differs), bf16 output
    against the exactly reconstructed weight at the 1e-2 bar; the float32
    output's distance from the exact-weight product is measured and reported
    (one bf16 rounding per weight: about 2^-9 / sqrt(3) = 1.1e-3)."""
    wl = synth.make(3)
    x, w, s, b, _ = synth.to_device(wl)
    want_tile = C.qmm(wl.x, wl.w, wl.scales, wl.biases, 64, 8, "affine", round_tile_bf16=True)
    want_exact = C.qmm(wl.x, wl.w, wl.scales, wl.biases, 64, 8, "affine", round_tile_bf16=False)
    y32 = out_f32(K.quantized_matmul(x, w, s, b, group_size=64, bits=8, out_dtype=torch.float32))
    y16 = out_f32(K.quantized_matmul(x, w, s, b, group_size=64, bits=8))
    d_tile, d_exact, d16 = O.rel_l2(y32, want_tile), O.rel_l2(y32, want_exact), O.rel_l2(y16, want_exact)
    _report("C3 full size", f32_vs_bf16_tile=d_tile, f32_vs_exact_weight=d_exact, bf16_vs_exact_weight=d16)
    assert d_tile <= 2e-5
    assert d_exact <= 3e-3
    assert d16 <= TOL_BF16_OUT
    np.testing.assert_array_equal(y16, O.round_bf16(y32))


def test_c4_mxfp4_full_size_against_the_oracle():
    """C4 whole (x [256, 8192] x MXFP4 [8192, 8192]) against the C oracle on the
    exact weight (E2M1 x 2^e is exact in every float type)."""
    wl = synth.make(4)
    x, w, s, _, _ = synth.to_device(wl)
    want = C.qmm(wl.x, wl.w, wl.scales, None, 32, 4, "mxfp4", round_tile_bf16=False)
    y32 = out_f32(K.quantized_matmul(x, w, s, None, group_size=32, bits=4, mode="mxfp4",
                                     out_dtype=torch.float32))
    y16 = out_f32(K.quantized_matmul(x, w, s, None, group_size=32, bits=4, mode="mxfp4"))
    d32, d16 = O.rel_l2(y32, want), O.rel_l2(y16, want)
    _report("C4 full size", f32_vs_exact_weight=d32, bf16_vs_exact_weight=d16)
    assert d32 <= TOL_F32_OUT
    assert d16 <= TOL_BF16_OUT


def test_c5_moe_full_size_against_the_oracle():
    """C5 whole (1024 routed rows, 8 experts of int4 g64 [14336, 4096]): the
    sorted-rows form in float32 and bf16, expert by expert, and the gathered
    form on the unsorted (token, expert) pairs of the same routing."""
    wl = synth.make(5)
    x, w, s, b, ro = synth.to_device(wl)
    ro_h = wl.row_offsets
    assert wl.x.shape == (1024, 4096) and wl.w.shape == (8, 14336, 512)
    want_tile = C.grouped_qmm(wl.x, wl.w, wl.scales, wl.biases, ro_h, 64, 4, "affine", round_tile_bf16=True)
    want_exact = C.grouped_qmm(wl.x, wl.w, wl.scales, wl.biases, ro_h, 64, 4, "affine", round_tile_bf16=False)
    y32 = out_f32(K.grouped_qmm(x, w, s, b, ro, group_size=64, bits=4, out_dtype=torch.float32))
    y16 = out_f32(K.grouped_qmm(x, w, s, b, ro, group_size=64, bits=4))
    for e in range(8):
        lo, hi = ro_h[e], ro_h[e + 1]
        assert hi > lo
        assert O.rel_l2(y32[lo:hi], want_tile[lo:hi]) <= 2e-5, e
        assert O.rel_l2(y16[lo:hi], want_exact[lo:hi]) <= TOL_BF16_OUT, e
    _report("C5 full size", f32_vs_bf16_tile=O.rel_l2(y32, want_tile),
            f32_vs_exact_weight=O.rel_l2(y32, want_exact), bf16_vs_exact_weight=O.rel_l2(y16, want_exact))
    assert O.rel_l2(y32, want_exact) <= 3e-3
    np.testing.assert_array_equal(y16, O.round_bf16(y32))
    # gathered form: pair p = 2 * token + j reads x_tokens[token] and expert experts[token, j];
    # sorted row r holds pair pair_of_row[r]
    ex = wl.extras
    tokens = ex["tokens"]
    xt = torch.from_numpy(ex["x_tokens"].view(np.int16)).to(DEV).view(torch.bfloat16)
    lhs = torch.arange(tokens, dtype=torch.int32, device=DEV).repeat_interleave(2)
    rhs = torch.from_numpy(ex["experts"].reshape(-1)).to(DEV)
    yg = out_f32(K.gather_qmm(xt, w, s, b, lhs, rhs, group_size=64, bits=4, out_dtype=torch.float32))
    assert yg.shape == (1024, 14336)
    np.testing.assert_array_equal(yg[ex["pair_of_row"]], y32)       # row for row the same arithmetic
    assert O.rel_l2(yg[ex["pair_of_row"]], want_tile) <= 2e-5


@pytest.mark.parametrize("bits,gs,k,mode", [
    (4, 64, 4352, "affine"),     # 68 entries a row: 136 bytes
    (4, 32, 2304, "affine"),     # 72 entries
    (8, 64, 4352, "affine"),
    (8, 32, 2304, "affine"),
    (4, 32, 4352, "mxfp4"),      # 136 scale bytes a row, K % 512 != 0: the bf16 kernels
])
def test_grouped_qmm_short_experts_with_table_rows_longer_than_a_cache_line(bits, gs, k, mode):
    """The split-role kernel stages a tile's scale / bias rows in LDS only when
    a row's table fits one 128-byte line; longer rows (these) take the 16-byte
    windows per quad of K-tiles instead."""
    rng = np.random.default_rng(bits * 1000 + gs + k)
    sizes = np.array([130, 0, 96, 161, 17])
    e, n = len(sizes), 136
    if mode == "affine":
        _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs, lead=(e,))
    else:
        _, words, s, wd, sd = make_mxfp4(rng, n, k, lead=(e,))
        b, bd = None, None
    ro = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    r = int(ro[-1])
    assert k % 256 == 0
    x, xd = make_x(rng, r, k)
    want = O.grouped_qmm(x, words, s, b, ro, gs, bits, mode, weight_rounding="bf16")
    ro_d = torch.from_numpy(ro).to(DEV)
    y32 = out_f32(K.grouped_qmm(xd, wd, sd, bd, ro_d, group_size=gs, bits=bits, mode=mode,
                                out_dtype=torch.float32))
    y16 = out_f32(K.grouped_qmm(xd, wd, sd, bd, ro_d, group_size=gs, bits=bits, mode=mode))
    for i in range(e):
        lo, hi = ro[i], ro[i + 1]
        if hi > lo:
            assert O.rel_l2(y32[lo:hi], want[lo:hi]) <= 2e-5, (i, O.rel_l2(y32[lo:hi], want[lo:hi]))
            assert O.rel_l2(y16[lo:hi], want[lo:hi]) <= TOL_BF16_OUT, i
    np.testing.assert_array_equal(y16, O.round_bf16(y32))


# ------------------------------------------ float16 / float32 activations ----

def _x_of(rng, m, k, el):
    x = rng.standard_normal((m, k)).astype(np.float32)
    if el == "f16":
        x = x.astype(np.float16)
        return x.astype(np.float32), torch.from_numpy(x).to(DEV)
    return x, torch.from_numpy(x).to(DEV)


@pytest.mark.parametrize("el", ["f32", "f16"])
@pytest.mark.parametrize("bits,gs,m,n,k", [
    (4, 64, 1, 300, 4096),      # three / two terms as rows of one decode launch (loader-wavefront kernel)
    (4, 64, 5, 2100, 4096),     # float32: 15 rows, still one decode launch
    (8, 64, 3, 200, 512),       # the self-loading kernel
    (4, 32, 2, 72, 96),         # the general decode kernel
    (4, 64, 8, 136, 1024),      # float32: 24 stacked rows -> the prefill kernel; float16: 16 -> decode
    (4, 128, 40, 200, 512),     # prefill
    (8, 64, 130, 136, 1024),
])
def test_float16_and_float32_activations_affine(el, bits, gs, m, n, k):
    """Activations wider than bf16 are split exactly into bf16 terms, so the
    product keeps the accuracy of the kernel that runs it: the exactly
    reconstructed weight where the stacked rows fit the decode kernel, the
    bf16-rounded weight tile on the prefill kernels."""
    rng = np.random.default_rng(bits * 100 + gs + m + k)
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, bits, gs)
    x, xd = _x_of(rng, m, k, el)
    terms = 3 if el == "f32" else 2
    rounding = "f32" if terms * m <= 16 else "bf16"
    want = O.qmm(x, words, s, b, gs, bits, weight_rounding=rounding)
    y32 = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits, out_dtype=torch.float32))
    assert O.rel_l2(y32, want) <= 2e-5, O.rel_l2(y32, want)
    y = K.quantized_matmul(xd, wd, sd, bd, group_size=gs, bits=bits)        # result in the activations' type
    assert y.dtype == xd.dtype
    assert O.rel_l2(out_f32(y), want) <= (2e-5 if el == "f32" else 1e-3)


@pytest.mark.parametrize("el", ["f32", "f16"])
@pytest.mark.parametrize("m,n,k", [(2, 72, 256), (4, 1200, 4096), (64, 136, 1024), (40, 200, 768)])
def test_float16_and_float32_activations_mxfp4(el, m, n, k):
    """MXFP4 weights are exact in bf16, so with exact activation terms the
    whole product is float32-accurate on every path (the reference's float32
    cases, tests/test_qmm_mxfp4.py:453: rtol 1e-5)."""
    rng = np.random.default_rng(m + n + k)
    _, words, sb, wd, sd = make_mxfp4(rng, n, k)
    x, xd = _x_of(rng, m, k, el)
    want = O.qmm(x, words, sb, None, 32, 4, "mxfp4")
    y32 = out_f32(K.quantized_matmul(xd, wd, sd, None, group_size=32, bits=4, mode="mxfp4",
                                     out_dtype=torch.float32))
    assert O.rel_l2(y32, want) <= 2e-5, O.rel_l2(y32, want)


def test_float32_activations_batched():
    rng = np.random.default_rng(11)
    bsz, m, n, k = 3, 2, 96, 512
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64, lead=(bsz,))
    x = rng.standard_normal((bsz, m, k)).astype(np.float32)
    xd = torch.from_numpy(x).to(DEV)
    want = np.stack([O.qmm(x[i], words[i], s[i], b[i], 64, 4) for i in range(bsz)])
    y = out_f32(K.quantized_matmul(xd, wd, sd, bd, group_size=64, bits=4))
    assert y.shape == (bsz, m, n)
    assert O.rel_l2(y, want) <= 2e-5, O.rel_l2(y, want)


@pytest.mark.parametrize("el", ["f32", "f16"])
def test_float16_and_float32_activations_grouped_and_gathered(el):
    """The expert-indexed forms on wider activations: one product per bf16
    term; rows outside the offsets and pairs naming no expert stay untouched."""
    rng = np.random.default_rng(5 + len(el))
    e, n, k = 4, 136, 512
    _, words, s, b, wd, sd, bd = make_affine(rng, n, k, 4, 64, lead=(e,))
    sizes = np.array([70, 0, 33, 20])
    ro = np.concatenate([[3], 3 + np.cumsum(sizes)]).astype(np.int32)     # rows 0-2 and the last four belong to no expert
    r = int(ro[-1]) + 4
    x, xd = _x_of(rng, r, k, el)
    want = O.grouped_qmm(x, words, s, b, ro, 64, 4, weight_rounding="bf16")
    given = torch.full((r, n), 7.0, dtype=torch.float32, device=DEV)
    K.grouped_qmm(xd, wd, sd, bd, torch.from_numpy(ro).to(DEV), group_size=64, bits=4, out=given)
    got = out_f32(given)
    assert (got[:3] == 7.0).all() and (got[ro[-1]:] == 7.0).all()
    assert O.rel_l2(got[3:ro[-1]], want[3:ro[-1]]) <= 2e-5
    # gathered: many pairs (prefill kernels), few pairs (grouped decode), three pairs (independent products)
    for pairs, rounding in ((300, "bf16"), (24, "f32"), (3, "f32")):
        lhs = rng.integers(0, r, size=pairs).astype(np.int32)
        rhs = rng.integers(0, e, size=pairs).astype(np.int32)
        rhs_dev = rhs.copy()
        rhs_dev[1] = e + 2                                   # names no expert
        wantg = O.gather_qmm(x[:, None, :], words, s, b, lhs, rhs, 64, 4, weight_rounding=rounding)[:, 0]
        yg = out_f32(K.gather_qmm(xd, wd, sd, bd, torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs_dev).to(DEV),
                                  group_size=64, bits=4, out_dtype=torch.float32))
        good = np.arange(pairs) != 1
        assert O.rel_l2(yg[good], wantg[good]) <= 2e-5, (pairs, O.rel_l2(yg[good], wantg[good]))
