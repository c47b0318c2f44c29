"""Seeded random sweep of the C ABI against the oracle: shapes, group sizes,
code widths, table types and output types drawn at random, so that every
kernel family and its edge handling (ragged tiles, short K, odd N, unaligned
table pitches) is hit by inputs nobody chose by hand."""
import numpy as np
import pytest
import torch

from metaljax_amd import kernels as K
from oracle import qmm_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _bf16_dev(v):
    return torch.from_numpy(np.ascontiguousarray(O.f32_to_bf16_bits(v)).view(np.int16)).to(DEV).view(torch.bfloat16)


def _tab_dev(v, tab):
    if tab == "bf16":
        return _bf16_dev(v)
    if tab == "f16":
        return torch.from_numpy(v.astype(np.float16)).to(DEV)
    return torch.from_numpy(v.astype(np.float32)).to(DEV)


def _draw_affine(rng):
    regime = rng.choice(["decode", "prefill", "prefill_big"])
    m = int(rng.integers(1, 17)) if regime == "decode" else int(rng.integers(17, 300 if regime == "prefill" else 700))
    n = int(rng.integers(1, 700))
    gs = int(rng.choice([32, 64, 128]))
    k = gs * int(rng.integers(1, 2048 // gs + 1))
    bits = int(rng.choice([4, 8]))
    tab = str(rng.choice(["bf16", "bf16", "f32", "f16"]))
    return m, n, k, gs, bits, tab


@pytest.mark.parametrize("seed", range(48))
def test_affine_random_case(seed):
    rng = np.random.default_rng(7000 + seed)
    m, n, k, gs, bits, tab = _draw_affine(rng)
    codes = rng.integers(0, 1 << bits, size=(n, k), dtype=np.uint8)
    words = O.pack_codes(codes, bits)
    s = rng.uniform(0.005, 0.02, (n, k // gs)).astype(np.float32)
    b = (-(rng.integers(0, 1 << bits, s.shape).astype(np.float32)) * s).astype(np.float32)
    if tab == "bf16":
        s, b = O.round_bf16(s), O.round_bf16(b)
    elif tab == "f16":
        s, b = s.astype(np.float16).astype(np.float32), b.astype(np.float16).astype(np.float32)
    x = O.round_bf16(rng.standard_normal((m, k)).astype(np.float32))
    wd = torch.from_numpy(np.ascontiguousarray(words).view(np.int32)).to(DEV)
    y = K.quantized_matmul(_bf16_dev(x), wd, _tab_dev(s, tab), _tab_dev(b, tab), group_size=gs, bits=bits,
                           out_dtype=torch.float32).float().cpu().numpy()
    rounding = "f32" if m <= 16 else "bf16"          # prefill stages a bf16 weight tile
    want = O.qmm(x, words, s, b, gs, bits, weight_rounding=rounding)
    err = O.rel_l2(y, want)
    assert err <= 2e-5, (m, n, k, gs, bits, tab, err)


@pytest.mark.parametrize("seed", range(16))
def test_mxfp4_random_case(seed):
    rng = np.random.default_rng(9000 + seed)
    m = int(rng.choice([int(rng.integers(1, 17)), int(rng.integers(17, 400))]))
    n = int(rng.integers(1, 500))
    k = 32 * int(rng.integers(1, 65))
    codes = rng.integers(0, 16, size=(n, k), dtype=np.uint8)
    words = O.pack_codes(codes, 4)
    sb = rng.integers(112, 140, size=(n, k // 32)).astype(np.uint8)
    x = O.round_bf16(rng.standard_normal((m, k)).astype(np.float32))
    wd = torch.from_numpy(np.ascontiguousarray(words).view(np.int32)).to(DEV)
    y = K.quantized_matmul(_bf16_dev(x), wd, torch.from_numpy(sb).to(DEV), None, group_size=32, bits=4,
                           mode="mxfp4", out_dtype=torch.float32).float().cpu().numpy()
    want = O.qmm(x, words, sb, None, 32, 4, "mxfp4")
    # K % 512 == 0 and M > 16 runs on the block-scaled matrix cores (two FP6 activation terms)
    tol = 1e-3 if (m > 16 and k % 512 == 0) else 2e-5
    err = O.rel_l2(y, want)
    assert err <= tol, (m, n, k, err)


@pytest.mark.parametrize("seed", range(12))
def test_grouped_and_gathered_random_case(seed):
    rng = np.random.default_rng(11000 + seed)
    e = int(rng.integers(1, 7))
    n = int(rng.integers(8, 300))
    gs = int(rng.choice([32, 64, 128]))
    k = gs * int(rng.integers(1, 1024 // gs + 1))
    bits = int(rng.choice([4, 8]))
    sizes = rng.integers(0, 200, size=e)
    sizes[rng.integers(0, e)] += 70                   # never all empty; total well past the decode regime
    ro = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    r = int(ro[-1])
    codes = rng.integers(0, 1 << bits, size=(e, n, k), dtype=np.uint8)
    words = O.pack_codes(codes, bits)
    s = O.round_bf16(rng.uniform(0.005, 0.02, (e, n, k // gs)).astype(np.float32))
    b = O.round_bf16(-(rng.integers(0, 1 << bits, s.shape).astype(np.float32)) * s)
    x = O.round_bf16(rng.standard_normal((r, k)).astype(np.float32))
    wd = torch.from_numpy(np.ascontiguousarray(words).view(np.int32)).to(DEV)
    sd, bd, xd = _bf16_dev(s), _bf16_dev(b), _bf16_dev(x)
    want = O.grouped_qmm(x, words, s, b, ro, gs, bits, weight_rounding="bf16")
    y = K.grouped_qmm(xd, wd, sd, bd, torch.from_numpy(ro).to(DEV), group_size=gs, bits=bits,
                      out_dtype=torch.float32).float().cpu().numpy()
    assert O.rel_l2(y, want) <= 2e-5, (e, n, k, gs, bits, sizes, O.rel_l2(y, want))
    # the same rows as shuffled (row, expert) pairs
    rhs = np.repeat(np.arange(e), sizes).astype(np.int32)
    perm = rng.permutation(r)
    yg = K.gather_qmm(xd, wd, sd, bd, torch.from_numpy(perm.astype(np.int32)).to(DEV),
                      torch.from_numpy(rhs[perm]).to(DEV), group_size=gs, bits=bits,
                      out_dtype=torch.float32).float().cpu().numpy()
    assert O.rel_l2(yg, want[perm]) <= 2e-5, (e, n, k, gs, bits, O.rel_l2(yg, want[perm]))


@pytest.mark.parametrize("seed", range(10))
def test_grouped_short_experts_random_case(seed):
    """Grouped products that run on the split-role kernel (bf16 tables,
    K % 256 == 0): many experts, empty ones, experts on either side of the
    borders between its three loops (128, 160 and 256 rows a tile) and past
    one tile, any N (also below one column tile and not a multiple of 8),
    every output type."""
    rng = np.random.default_rng(12000 + seed)
    e = int(rng.integers(1, 13))
    n = int(rng.choice([rng.integers(1, 128), rng.integers(128, 400)]))
    gs = int(rng.choice([32, 64, 128]))
    k = 256 * int(rng.integers(1, 5))
    bits = int(rng.choice([4, 8]))
    sizes = rng.integers(0, 150, size=e)
    sizes[rng.integers(0, e)] += int(rng.choice([20, 120, 200]))
    if seed % 2:
        sizes[rng.integers(0, e)] += int(rng.choice([60, 110, 260]))
    ro = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    r = int(ro[-1])
    codes = rng.integers(0, 1 << bits, size=(e, n, k), dtype=np.uint8)
    words = O.pack_codes(codes, bits)
    s = O.round_bf16(rng.uniform(0.005, 0.02, (e, n, k // gs)).astype(np.float32))
    b = O.round_bf16(-(rng.integers(0, 1 << bits, s.shape).astype(np.float32)) * s)
    x = O.round_bf16(rng.standard_normal((r, k)).astype(np.float32))
    wd = torch.from_numpy(np.ascontiguousarray(words).view(np.int32)).to(DEV)
    sd, bd, xd = _bf16_dev(s), _bf16_dev(b), _bf16_dev(x)
    want = O.grouped_qmm(x, words, s, b, ro, gs, bits, weight_rounding="bf16")
    out_dtype = [torch.float32, torch.bfloat16, torch.float16][seed % 3]
    tol = 2e-5 if out_dtype == torch.float32 else (1e-2 if out_dtype == torch.bfloat16 else 2e-3)
    y = K.grouped_qmm(xd, wd, sd, bd, torch.from_numpy(ro).to(DEV), group_size=gs, bits=bits,
                      out_dtype=out_dtype).float().cpu().numpy()
    assert y.shape == want.shape
    if r:
        assert O.rel_l2(y, want) <= tol, (e, n, k, gs, bits, sizes, O.rel_l2(y, want))
        for lo, hi in zip(ro[:-1], ro[1:]):
            if hi > lo:
                assert O.rel_l2(y[lo:hi], want[lo:hi]) <= tol, (lo, hi)


@pytest.mark.parametrize("seed", range(12))
def test_one_pass_decode_random_case(seed):
    """Decode shapes whose K is exactly one pass of eight 256-byte slices (the
    kernel whose compute wavefronts fetch their own activations when M <= 8):
    any number of tiles a workgroup, ragged last tiles, several rounds of
    workgroups, a leading batch axis, both output types."""
    rng = np.random.default_rng(9100 + seed)
    bits = int(rng.choice([4, 8]))
    k = 4096 if bits == 4 else 2048
    gs = int(rng.choice([64, 128]))
    m = int(rng.integers(1, 13))                       # above 8 the ring variant takes over
    n = int(rng.choice([rng.integers(16, 600), rng.integers(600, 9000), rng.integers(9000, 36000)]))
    batch = int(rng.choice([1, 1, 2])) if n < 9000 else 1
    lead = (batch,) if batch > 1 else ()
    codes = rng.integers(0, 1 << bits, size=lead + (n, k), dtype=np.uint8)
    words = O.pack_codes(codes, bits)
    s = O.round_bf16(rng.uniform(0.005, 0.02, lead + (n, k // gs)).astype(np.float32))
    b = O.round_bf16(-(rng.integers(0, 1 << bits, s.shape).astype(np.float32)) * s)
    x = O.round_bf16(rng.standard_normal(lead + (m, k)).astype(np.float32))
    wd = torch.from_numpy(np.ascontiguousarray(words).view(np.int32)).to(DEV)
    y32 = K.quantized_matmul(_bf16_dev(x), wd, _bf16_dev(s), _bf16_dev(b), group_size=gs, bits=bits,
                             out_dtype=torch.float32).float().cpu().numpy()
    want = O.qmm(x, words, s, b, gs, bits)
    err = O.rel_l2(y32, want)
    assert err <= 2e-5, (m, n, k, gs, bits, batch, err)
    y16 = K.quantized_matmul(_bf16_dev(x), wd, _bf16_dev(s), _bf16_dev(b), group_size=gs, bits=bits)
    np.testing.assert_array_equal(y16.float().cpu().numpy(), O.round_bf16(y32))


@pytest.mark.parametrize("seed", range(32))
def test_big_decode_random_case(seed):
    """Decode shapes with at least eight 256-byte K-slices, drawn at random over
    everything the loader-wavefront kernel distinguishes: passes over K (one to
    four, the last possibly part full), rows of activations (row packing or a
    fetch per pass), tiles a workgroup, code width, group size, bf16 / float16
    tables, MXFP4, a batch axis."""
    rng = np.random.default_rng(12000 + seed)
    kind = str(rng.choice(["int4", "int4", "int8", "mxfp4"]))
    bits = 8 if kind == "int8" else 4
    slice_k = 2048 // bits                                   # codes in a 256-byte slice
    slices = int(rng.integers(8, 33))
    k = slices * slice_k
    if kind == "mxfp4":
        k = max(4096, k // 512 * 512)
    m = int(rng.integers(1, 17))
    n = int(rng.choice([rng.integers(16, 400), rng.integers(400, 6000), rng.integers(6000, 30000)]))
    if n * k > 120_000_000:                                  # keep the oracle's float64 product quick
        n = 120_000_000 // k
    batch = 2 if (n * k < 8_000_000 and rng.random() < 0.3) else 1
    lead = (batch,) if batch > 1 else ()
    x = O.round_bf16(rng.standard_normal(lead + (m, k)).astype(np.float32))
    codes = rng.integers(0, 1 << bits, size=lead + (n, k), dtype=np.uint8)
    words = O.pack_codes(codes, bits)
    wd = torch.from_numpy(np.ascontiguousarray(words).view(np.int32)).to(DEV)
    if kind == "mxfp4":
        sb = rng.integers(110, 140, size=lead + (n, k // 32)).astype(np.uint8)
        y = K.quantized_matmul(_bf16_dev(x), wd, torch.from_numpy(sb).to(DEV), None, group_size=32, bits=4,
                               mode="mxfp4", out_dtype=torch.float32).float().cpu().numpy()
        want = O.qmm(x, words, sb, None, 32, 4, "mxfp4")
        info = (kind, m, n, k, batch)
    else:
        gs = int(rng.choice([64, 128]))
        tab = str(rng.choice(["bf16", "bf16", "f16"]))
        s = rng.uniform(0.005, 0.02, lead + (n, k // gs)).astype(np.float32)
        b = -(rng.integers(0, 1 << bits, s.shape).astype(np.float32)) * s
        if tab == "bf16":
            s, b = O.round_bf16(s), O.round_bf16(b)
        else:
            s, b = s.astype(np.float16).astype(np.float32), b.astype(np.float16).astype(np.float32)
        y = K.quantized_matmul(_bf16_dev(x), wd, _tab_dev(s, tab), _tab_dev(b, tab), group_size=gs, bits=bits,
                               out_dtype=torch.float32).float().cpu().numpy()
        want = O.qmm(x, words, s, b, gs, bits)
        info = (kind, gs, tab, m, n, k, batch)
    err = O.rel_l2(y, want)
    assert err <= 2e-5, (info, err)


@pytest.mark.parametrize("seed", range(12))
def test_grouped_decode_random_case(seed):
    """Expert-indexed products with few pairs (4 <= P <= 16 E): random routing,
    skewed or not, with indices that name no expert or no row now and then."""
    rng = np.random.default_rng(13000 + seed)
    kind = str(rng.choice(["int4", "int8", "mxfp4"]))
    bits = 8 if kind == "int8" else 4
    k = int(rng.choice([1, 2, 3])) * (4096 if bits == 4 else 2048)
    e = int(rng.integers(1, 9))
    n = int(rng.integers(16, 3000))
    t = int(rng.integers(1, 40))
    pairs = int(rng.integers(4, 16 * e + 1))
    lhs = rng.integers(0, t, size=pairs).astype(np.int32)
    rhs = rng.integers(0, e, size=pairs).astype(np.int32)
    if rng.random() < 0.5:
        rhs[rng.random(pairs) < 0.7] = int(rng.integers(0, e))
    x = O.round_bf16(rng.standard_normal((t, k)).astype(np.float32))
    codes = rng.integers(0, 1 << bits, size=(e, n, k), dtype=np.uint8)
    words = O.pack_codes(codes, bits)
    wd = torch.from_numpy(np.ascontiguousarray(words).view(np.int32)).to(DEV)
    ld, rd = torch.from_numpy(lhs).to(DEV), torch.from_numpy(rhs).to(DEV)
    if kind == "mxfp4":
        sb = rng.integers(110, 140, size=(e, n, k // 32)).astype(np.uint8)
        y = K.gather_qmm(_bf16_dev(x), wd, torch.from_numpy(sb).to(DEV), None, ld, rd, group_size=32, bits=4,
                         mode="mxfp4", out_dtype=torch.float32).float().cpu().numpy()
        want = O.gather_qmm(x[:, None, :], words, sb, None, lhs, rhs, 32, 4, "mxfp4")[:, 0]
    else:
        s = O.round_bf16(rng.uniform(0.005, 0.02, (e, n, k // 64)).astype(np.float32))
        b = O.round_bf16(-(rng.integers(0, 1 << bits, s.shape).astype(np.float32)) * s)
        y = K.gather_qmm(_bf16_dev(x), wd, _bf16_dev(s), _bf16_dev(b), ld, rd, group_size=64, bits=bits,
                         out_dtype=torch.float32).float().cpu().numpy()
        want = O.gather_qmm(x[:, None, :], words, s, b, lhs, rhs, 64, bits)[:, 0]
    err = O.rel_l2(y, want)
    assert err <= 2e-5, (kind, k, e, n, t, pairs, err)
