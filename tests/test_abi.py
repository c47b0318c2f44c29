"""The C-ABI library: it loads, exports every function include/qmm_hip.h
declares, and its host-only entry points (no device work) behave.  Runs
without a GPU; no compute entry point is called here."""

import ctypes
import os
import re

import pytest

from metaljax_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "qmm_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return sorted(set(re.findall(r"\b(qmm_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        from metaljax_amd import build
        build.build()
    return _lib.load()


def test_header_and_binding_agree():
    assert declared_functions() == sorted(_lib.SYMBOLS)


def test_library_exports_every_declared_symbol(lib):
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(raw, name), name


def test_header_cites_the_reference_for_every_entry_point():
    text = open(HEADER).read()
    # each declaration is preceded by a comment naming the reference call it replaces
    for name in declared_functions():
        if name in ("qmm_abi_version", "qmm_last_error", "qmm_workspace_bytes",
                    "qmm_gather_workspace_bytes", "qmm_plan"):
            continue
        if name == "qmm_gather_qmm_static":      # says that the reference has no such call
            head = text[:text.index(name + "(")]
            assert "No counterpart in the reference" in head[head.rindex("/*"):]
            continue
        head = text[:text.index(name + "(")]
        comment = head[head.rindex("/*"):]
        assert re.search(r"\.py:\d+", comment), f"{name}: no reference citation"


def test_abi_version_and_error_text(lib):
    assert lib.qmm_abi_version() >= 1
    assert isinstance(lib.qmm_last_error(), bytes)


def test_plan_picks_the_regime(lib):
    k, g, b = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    assert lib.qmm_plan(1, 4096, 4096, 64, 4, 0, k, g, b) == 0
    assert k.value == _lib.KERNEL_GEMV and g.value > 0 and b.value % 64 == 0
    assert lib.qmm_plan(16, 14336, 4096, 64, 4, 0, k, g, b) == 0
    assert k.value == _lib.KERNEL_GEMV
    assert lib.qmm_plan(2048, 4096, 4096, 64, 8, 0, k, g, b) == 0
    assert k.value == _lib.KERNEL_GEMM and g.value >= 256


def test_plan_of_the_decode_variants(lib):
    """The decode plan follows the kernel choice: 768-thread workgroups (eight
    compute + four loader wavefronts) where the loader-wavefront kernel serves
    the shape, one workgroup per compute unit (256 assumed without a device)
    with up to 128 rows each when the activations are fetched directly."""
    k, g, b = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    assert lib.qmm_plan(4, 28672, 4096, 64, 4, 0, k, g, b) == 0
    assert (k.value, b.value) == (_lib.KERNEL_GEMV, 768)
    rows = -(-28672 // g.value)
    assert 16 <= rows <= 128 and g.value * rows >= 28672
    assert lib.qmm_plan(16, 14336, 4096, 64, 4, 0, k, g, b) == 0        # ring variant: at most 64 rows
    assert b.value == 768 and -(-14336 // g.value) <= 64
    assert lib.qmm_plan(4, 4096, 1024, 64, 4, 0, k, g, b) == 0          # two slices: the self-loading kernel
    assert k.value == _lib.KERNEL_GEMV and b.value < 768
    assert lib.qmm_plan(4, 16384, 3072, 64, 4, 0, k, g, b) == 0         # six slices: loader wavefronts again
    assert k.value == _lib.KERNEL_GEMV and b.value == 768
    assert lib.qmm_plan(16, 3072, 3072, 64, 4, 0, k, g, b) == 0         # ... at sixteen rows too
    assert b.value == 768


def test_plan_of_the_mxfp4_kernels(lib):
    """MXFP4 prefill: the eight-wavefront block-scaled kernel (512 threads, a
    64 x 128 tile a workgroup) when K is a whole number of 2048-code stages,
    the four-wavefront one for the other multiples of 512, the bf16 kernels
    otherwise.  MXFP4 decode: the loader-wavefront kernel (768 threads) from
    three 512-code slices a row on, for a K that is no whole number of slices
    (gpt-oss: 2880) its one-pass form with rows dealt by eights."""
    k, g, b = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    assert lib.qmm_plan(256, 8192, 8192, 32, 4, 1, k, g, b) == 0
    assert (k.value, g.value, b.value) == (_lib.KERNEL_MXFP4_MFMA, (8192 // 128) * (256 // 64), 512)
    assert lib.qmm_plan(300, 260, 1536, 32, 4, 1, k, g, b) == 0
    assert (k.value, b.value) == (_lib.KERNEL_MXFP4_MFMA, 256) and g.value == 16      # 3 x 5 tiles, dealt to eight XCDs
    assert lib.qmm_plan(256, 5760, 2880, 32, 4, 1, k, g, b) == 0        # K % 512 != 0: the bf16 prefill kernel
    assert k.value == _lib.KERNEL_GEMM
    for m in (1, 16):
        assert lib.qmm_plan(m, 5760, 2880, 32, 4, 1, k, g, b) == 0
        rows = -(-5760 // g.value)
        assert (k.value, b.value) == (_lib.KERNEL_GEMV, 768) and rows % 8 == 0 and 16 <= rows <= 128
        assert lib.qmm_plan(m, 8192, 8192, 32, 4, 1, k, g, b) == 0
        assert (k.value, b.value) == (_lib.KERNEL_GEMV, 768) and g.value == 256
    assert lib.qmm_plan(4, 4096, 1024, 32, 4, 1, k, g, b) == 0          # two slices: the general decode kernel
    assert k.value == _lib.KERNEL_GEMV and b.value < 768
    assert lib.qmm_plan(4, 4096, 4160, 32, 4, 1, k, g, b) == 0          # ragged beyond eight slices: general again
    assert b.value < 768
    assert lib.qmm_plan(4, 100, 2880, 32, 4, 1, k, g, b) == 0           # an expert's scale table no multiple of 16 bytes
    assert b.value < 768


def test_gather_workspace_covers_the_grouped_decode(lib):
    """From four pairs up to sixteen an expert the workspace holds the expert
    sort and the segment list; below four pairs nothing is needed."""
    assert lib.qmm_gather_workspace_bytes(2, 8, 14336, 4096, _lib.BF16) == 0
    few = lib.qmm_gather_workspace_bytes(16, 8, 14336, 4096, _lib.BF16)
    sort_only = ((2 * 8 + 1 + 2 * 16) * 4 + 255) // 256 * 256
    assert few >= sort_only and few % 256 == 0
    assert lib.qmm_gather_workspace_bytes(128, 8, 14336, 4096, _lib.BF16) >= lib.qmm_gather_workspace_bytes(16, 8, 14336, 4096, _lib.BF16)


def test_workspace_queries_need_no_device(lib):
    assert lib.qmm_workspace_bytes(1, 16, 14336, 4096, 64, 4, 0, _lib.BF16) == 0
    need = lib.qmm_gather_workspace_bytes(1024, 8, 14336, 4096, _lib.BF16)
    assert need > 0 and need % 4 == 0
    assert lib.qmm_gather_workspace_bytes(0, 8, 64, 64, _lib.BF16) >= 0


def test_argument_errors_are_reported_before_any_launch(lib):
    # null pointers / bad enums are rejected on the host (no GPU needed)
    rc = lib.qmm_quantized_matmul(None, _lib.BF16, None, None, None, _lib.BF16, None, _lib.BF16,
                                  1, 1, 64, 64, 64, 4, 0, None, 0, None)
    assert rc != 0
    assert lib.qmm_last_error()
    rc = lib.qmm_quantized_matmul(None, _lib.BF16, None, None, None, _lib.BF16, None, _lib.BF16,
                                  1, 1, 64, 48, 64, 4, 0, None, 0, None)
    assert rc in (1, 2, 3)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libqmm_hip.so"))
    with pytest.raises(_lib.QmmLibraryError):
        _lib.load()


def test_static_scratch_entry_point_rejects_what_does_not_fit(lib):
    """qmm_gather_qmm_static refuses, on the host and before any device work,
    a product whose scratch need exceeds the array built into the library."""
    text = open(HEADER).read()
    assert re.search(r"#define QMM_STATIC_SCRATCH_BYTES \(16u << 20\)", text)
    assert _lib.STATIC_SCRATCH_BYTES == 16 << 20
    p, e, n, k = 4096, 8, 14336, 4096                 # the re-laid activations alone are 32 MiB
    assert lib.qmm_gather_workspace_bytes(p, e, n, k, _lib.BF16) > _lib.STATIC_SCRATCH_BYTES
    rc = lib.qmm_gather_qmm_static(None, _lib.BF16, None, None, None, _lib.BF16, None, _lib.BF16,
                                   None, None, p, p, e, n, k, 64, 4, 0, None)
    assert rc == 4 and b"static scratch" in lib.qmm_last_error()
