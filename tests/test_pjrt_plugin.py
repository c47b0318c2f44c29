"""The PJRT plugin (`libqmm_pjrt.so`, GetPjrtApi over `metaljax_amd.engine`;
the role of the reference's plugin/metal_pjrt.cc) driven through the PJRT C
API by the C++ harness in tests/pjrt_harness.cc, which does what a framework's
client does: load, initialise, create a client, compile, move buffers in,
execute, move results out.  jax is not installed here, so no `jax.jit` program
runs through it ("parity unpinned" against a real JAX client); what is pinned
is the C API contract of every call the harness makes and that results equal
the engine's own.

Both libraries are built by `python -m metaljax_amd.build` against OpenXLA's
pjrt_c_api.h, which is not part of this tree: where neither the header nor a
built library is present the tests skip."""

import ctypes
import os

import numpy as np
import pytest

import stablehlo_text as T
from metaljax_amd import build as B, engine

PLUGIN, HARNESS = B.PJRT_LIB, B.PJRT_HARNESS
pytestmark = pytest.mark.skipif(not (os.path.exists(PLUGIN) and os.path.exists(HARNESS)),
                                reason="PJRT plugin not built (no pjrt_c_api.h at build time)")

F32 = engine.PJRT_TYPES.index("F32")
BF16 = engine.PJRT_TYPES.index("BF16")
UNIMPLEMENTED, INTERNAL, INVALID_ARGUMENT = 12, 13, 3        # PJRT_Error_Code values


class Harness:
    def __init__(self):
        h = ctypes.CDLL(HARNESS)
        i, p, c, i64p, ip = ctypes.c_int, ctypes.c_void_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int)
        h.pjrt_harness_last_error.restype = c
        h.pjrt_harness_open.argtypes = [c]
        h.pjrt_harness_info.argtypes = [ip, c, i, c, i, ip, i64p]
        h.pjrt_harness_compile.argtypes = [c, ctypes.c_int64, c, ip]
        h.pjrt_harness_executable_info.argtypes = [i, ip, ip, ip, i64p, i, c, i, c, i]
        h.pjrt_harness_buffer_from_host.argtypes = [p, i, i64p, i, i64p, ip]
        h.pjrt_harness_buffer_info.argtypes = [i, i64p, i64p]
        h.pjrt_harness_to_host.argtypes = [i, p, i64p]
        h.pjrt_harness_execute.argtypes = [i, ip, i, ip, i, ip]
        self.h = h
        self.ok(h.pjrt_harness_open(PLUGIN.encode()))

    def error(self):
        return self.h.pjrt_harness_last_error().decode(errors="replace")

    def ok(self, rc):
        assert rc == 0, (rc, self.error())

    def close(self):
        self.ok(self.h.pjrt_harness_close())

    def info(self):
        ver = (ctypes.c_int * 2)()
        counts = (ctypes.c_int * 2)()
        shlo = (ctypes.c_int64 * 3)()
        plat, kind = ctypes.create_string_buffer(64), ctypes.create_string_buffer(128)
        self.ok(self.h.pjrt_harness_info(ver, plat, 64, kind, 128, counts, shlo))
        return list(ver), plat.value.decode(), kind.value.decode(), list(counts), list(shlo)

    def compile(self, text, fmt="mlir"):
        raw = text if isinstance(text, bytes) else text.encode()
        out = ctypes.c_int(-1)
        rc = self.h.pjrt_harness_compile(raw, len(raw), fmt.encode(), ctypes.byref(out))
        return rc, out.value

    def executable_info(self, handle, cap=8):
        counts = (ctypes.c_int * 3)()
        types, ranks = (ctypes.c_int * cap)(), (ctypes.c_int * cap)()
        dims = (ctypes.c_int64 * (8 * cap))()
        name, fp = ctypes.create_string_buffer(64), ctypes.create_string_buffer(128)
        self.ok(self.h.pjrt_harness_executable_info(handle, counts, types, ranks, dims, cap, name, 64, fp, 128))
        n = counts[0]
        shapes, at = [], 0
        for r in list(ranks)[:n]:
            shapes.append(list(dims)[at:at + r])
            at += r
        return list(counts), list(types)[:n], shapes, name.value.decode(), fp.value.decode()

    def buffer(self, arr, type_enum, strides=None):
        dims = (ctypes.c_int64 * arr.ndim)(*arr.shape)
        st = None if strides is None else (ctypes.c_int64 * arr.ndim)(*strides)
        out = ctypes.c_int(-1)
        rc = self.h.pjrt_harness_buffer_from_host(arr.ctypes.data_as(ctypes.c_void_p), type_enum, dims, arr.ndim, st,
                                                  ctypes.byref(out))
        return rc, out.value

    def buffer_info(self, handle):
        info, dims = (ctypes.c_int64 * 6)(), (ctypes.c_int64 * 8)()
        self.ok(self.h.pjrt_harness_buffer_info(handle, info, dims))
        t, rank, nbytes, ptr, on_cpu, deleted = list(info)
        return dict(type=t, dims=list(dims)[:rank], nbytes=nbytes, pointer=ptr, on_cpu=bool(on_cpu), deleted=bool(deleted))

    def to_host(self, handle):
        size = ctypes.c_int64(0)
        self.ok(self.h.pjrt_harness_to_host(handle, None, ctypes.byref(size)))     # the size query
        raw = ctypes.create_string_buffer(max(1, size.value))
        rc = self.h.pjrt_harness_to_host(handle, raw, ctypes.byref(size))
        return rc, raw.raw[:size.value]

    def execute(self, exe, args, cap=8):
        a = (ctypes.c_int * len(args))(*args)
        outs, n = (ctypes.c_int * cap)(), ctypes.c_int(0)
        rc = self.h.pjrt_harness_execute(exe, a, len(args), outs, cap, ctypes.byref(n))
        return rc, list(outs)[:n.value]


@pytest.fixture()
def plugin():
    h = Harness()
    yield h
    h.close()


def test_the_api_table_is_complete_and_describes_one_device(plugin):
    """Every member of PJRT_Api is set (a framework calls through the table
    without checking), the version is the header's, and the client has one
    addressable device and one memory (reference metal_pjrt.cc:1276-1411)."""
    assert plugin.h.pjrt_harness_null_entries() == 0
    ver, platform, kind, counts, shlo = plugin.info()
    assert ver[0] == 0 and ver[1] >= 100
    assert platform == "qmm_hip"
    assert kind == engine.device_kind()
    assert counts == [1, 1]
    assert shlo == engine.stablehlo_version()
    # an entry point this plugin leaves out answers UNIMPLEMENTED
    assert plugin.h.pjrt_harness_topology() == UNIMPLEMENTED
    assert "does not implement" in plugin.error()


def test_compile_execute_and_copy_back_equal_the_engine(plugin):
    text = T.float_dot(8, 16, 4, el="f32")          # y = x @ (w * r[:, None])
    rc, exe = plugin.compile(text)
    plugin.ok(rc)
    ex = engine.compile_program(text.encode(), "mlir", None)
    counts, types, shapes, name, fp = plugin.executable_info(exe)
    assert counts == [1, 1, 1]                        # outputs, replicas, partitions
    assert types == ex.out_types == [F32] and shapes == ex.out_dims == [[4, 16]]
    assert name == ex.name and fp == ex.fingerprint
    rng = np.random.default_rng(0)
    w = rng.standard_normal((8, 16)).astype(np.float32)
    r = rng.standard_normal((8,)).astype(np.float32)
    x = rng.standard_normal((4, 8)).astype(np.float32)
    # w arrives as a strided (transposed) host view, as PJRT hands arrays over
    wt = np.ascontiguousarray(w.T)
    rc, bw = plugin.buffer(wt.T, F32, strides=[4, 4 * 8])
    plugin.ok(rc)
    (rc, br), (rc2, bx) = plugin.buffer(r, F32), plugin.buffer(x, F32)
    plugin.ok(rc), plugin.ok(rc2)
    info = plugin.buffer_info(bx)
    assert info["type"] == F32 and info["dims"] == [4, 8] and info["nbytes"] == x.nbytes
    assert info["pointer"] != 0 and not info["on_cpu"] and not info["deleted"]
    rc, raw = plugin.to_host(bw)
    plugin.ok(rc)
    assert raw == w.tobytes()                         # the strided view came in as the logical array
    rc, outs = plugin.execute(exe, [bw, br, bx])
    plugin.ok(rc)
    assert len(outs) == 1
    yinfo = plugin.buffer_info(outs[0])
    assert yinfo["type"] == F32 and yinfo["dims"] == [4, 16] and yinfo["nbytes"] == 4 * 16 * 4
    rc, raw = plugin.to_host(outs[0])
    plugin.ok(rc)
    want = engine.to_host(engine.execute(ex, [engine.buffer_from_host(memoryview(w), F32, [8, 16]),
                                              engine.buffer_from_host(memoryview(r), F32, [8]),
                                              engine.buffer_from_host(memoryview(x), F32, [4, 8])])[0])
    assert raw == want
    np.testing.assert_allclose(np.frombuffer(raw, np.float32).reshape(4, 16), x @ (w * r[:, None]), rtol=1e-5, atol=1e-5)
    # an output is a valid argument of the next execute; the caller's arrays are
    # free once BufferFromHostBuffer has returned (its event was ready)
    x[:] = 0
    rc, outs2 = plugin.execute(exe, [bw, br, bx])
    plugin.ok(rc)
    assert plugin.to_host(outs2[0])[1] == want


def test_the_smaller_entry_points_answer_as_the_c_api_says(plugin):
    """Events a caller creates and sets (deferred and immediate callbacks, an
    error handed on), a buffer's ready event, dense layout, copies, external
    reference counts, the memory's kind and user data, look-ups, the default
    device assignment, the loaded executable's device / fingerprint / memory
    kinds, and deletion: a scripted walk in the harness that reports the first
    step whose answer was not the C API's."""
    text = T.float_dot(8, 16, 4, el="f32")
    rc, exe = plugin.compile(text)
    plugin.ok(rc)
    rc, b = plugin.buffer(np.arange(24, dtype=np.float32).reshape(2, 3, 4), F32)
    plugin.ok(rc)
    step = plugin.h.pjrt_harness_walk(b, exe)
    assert step == 0, (step, plugin.error())
    plugin.ok(plugin.h.pjrt_harness_executable_delete(exe))
    rc, _ = plugin.execute(exe, [b, b, b])
    assert rc == INVALID_ARGUMENT and "deleted" in plugin.error()


def test_a_donated_parameter_is_consumed_unless_the_caller_keeps_it(plugin):
    """`jax.buffer_donor` / `tf.aliasing_output` on a parameter: the call
    consumes that buffer (reference metal_pjrt.cc:1032-1036, :1109-1116) unless
    the execute options list it as not donatable."""
    text = T.float_dot(8, 16, 4, el="f32").replace("%x: tensor<4x8xf32>", "%x: tensor<4x8xf32> {jax.buffer_donor = true}")
    assert engine.compile_program(text).donated_params == [2]
    rc, exe = plugin.compile(text)
    plugin.ok(rc)
    rng = np.random.default_rng(1)
    w, r, x = (rng.standard_normal(s).astype(np.float32) for s in ((8, 16), (8,), (4, 8)))
    (_, bw), (_, br), (_, bx) = plugin.buffer(w, F32), plugin.buffer(r, F32), plugin.buffer(x, F32)
    plugin.h.pjrt_harness_keep_inputs.argtypes = [ctypes.POINTER(ctypes.c_int64), ctypes.c_int]
    plugin.ok(plugin.h.pjrt_harness_keep_inputs((ctypes.c_int64 * 1)(2), 1))
    rc, outs = plugin.execute(exe, [bw, br, bx])
    plugin.ok(rc)
    assert not plugin.buffer_info(bx)["deleted"]          # kept
    rc, outs = plugin.execute(exe, [bw, br, bx])
    plugin.ok(rc)
    assert plugin.buffer_info(bx)["deleted"] and not plugin.buffer_info(bw)["deleted"]
    rc, raw = plugin.to_host(outs[0])
    plugin.ok(rc)
    np.testing.assert_allclose(np.frombuffer(raw, np.float32).reshape(4, 16), x @ (w * r[:, None]), rtol=1e-5, atol=1e-5)
    rc, _ = plugin.execute(exe, [bw, br, bx])              # a consumed buffer is not an argument any more
    assert rc == INVALID_ARGUMENT and "deleted" in plugin.error()


def test_bf16_bytes_round_trip(plugin):
    bits = np.array([0x3F80, 0xC000, 0x0000, 0x7F7F], np.uint16)
    rc, b = plugin.buffer(bits, BF16)
    plugin.ok(rc)
    assert plugin.buffer_info(b)["nbytes"] == 8
    rc, raw = plugin.to_host(b)
    plugin.ok(rc)
    assert raw == bits.tobytes()


def test_failures_come_back_as_errors_with_the_reference_codes(plugin):
    """A Python exception becomes a PJRT_Error with the traceback text; its
    code is UNIMPLEMENTED when the class name contains "Unsupported", else
    INTERNAL (reference metal_pjrt.cc:185-226); bad calls are INVALID_ARGUMENT."""
    rc, _ = plugin.compile("this is not a module")
    assert rc == INTERNAL and "compile_program" in plugin.error() and "Traceback" in plugin.error()
    rc, _ = plugin.compile(b"ML\xefR\x01StableHLO_v1.0.0")          # MLIR bytecode, and no jaxlib here to print it
    assert rc == UNIMPLEMENTED and "UnsupportedProgram" in plugin.error() and "jaxlib" in plugin.error()
    rc, _ = plugin.compile(T.float_dot(8, 16, 4, el="f32"), fmt="hlo")
    assert rc == UNIMPLEMENTED and "program format" in plugin.error()
    rc, _ = plugin.buffer(np.zeros(2, np.complex64), engine.PJRT_TYPES.index("C64"))
    assert rc == INTERNAL and "Unsupported PJRT buffer type" in plugin.error()     # a TypeError: the class decides
    rc, _ = plugin.buffer(np.zeros(2, np.uint8), engine.PJRT_TYPES.index("F8E5M2"))
    assert rc == UNIMPLEMENTED                                                        # no byte size known to the plugin
    text = T.float_dot(8, 16, 4, el="f32")
    rc, exe = plugin.compile(text)
    plugin.ok(rc)
    rc, b = plugin.buffer(np.zeros((4, 8), np.float32), F32)
    plugin.ok(rc)
    rc, _ = plugin.execute(exe, [b])                  # three parameters expected
    assert rc == INVALID_ARGUMENT and "number of arguments" in plugin.error()
    plugin.ok(plugin.h.pjrt_harness_buffer_delete(b))
    assert plugin.buffer_info(b)["deleted"]
    rc = plugin.h.pjrt_harness_to_host(b, None, ctypes.byref(ctypes.c_int64(0)))
    assert rc == INVALID_ARGUMENT and "deleted" in plugin.error()
    plugin.ok(plugin.h.pjrt_harness_buffer_destroy(b))


@pytest.mark.gpu
def test_a_recognized_quantized_dot_through_the_plugin():
    """The hot path end to end behind the C API: a sub-channel int4 program is
    compiled through PJRT_Client_Compile, its weights arrive through
    BufferFromHostBuffer, Execute runs the recognizer's fused HIP kernel, and
    the bytes that ToHostBuffer copies out equal what the engine returns when
    called directly."""
    import torch
    from metaljax_amd import interpreter as I, qmm
    assert torch.cuda.is_available()
    qmm.reset_stats()
    qmm._BUILT.clear()
    qmm._SHARED.clear()
    k, n, m = 256, 128, 4
    q, packed, scale, zero, g_idx, wref = T.quantize(k, n, 64, seed=7)
    x = T.bf16_round(np.random.default_rng(3).standard_normal((m, k)).astype(np.float32) * 0.5)
    text = T.dense_sub(k, n, scale.shape[0], m)
    from metaljax_amd.packing import f32_to_bf16_bits
    plugin = Harness()
    try:
        rc, exe = plugin.compile(text)
        plugin.ok(rc)
        ex = engine.compile_program(text)
        host_args = [packed, f32_to_bf16_bits(scale), zero, g_idx, f32_to_bf16_bits(x)]
        enums = [engine._EL_ENUM[a.type.el] for a in ex.interp.main.body.args]
        handles = []
        for arr, en in zip(host_args, enums):
            arr = np.ascontiguousarray(arr)
            rc, h = plugin.buffer(arr, en)
            plugin.ok(rc)
            handles.append(h)
        rc, outs = plugin.execute(exe, handles)
        plugin.ok(rc)
        st = qmm.stats()
        assert st["packs"] == 1 and st["fallbacks"] == 0          # the fused kernel ran, not the literal chain
        info = plugin.buffer_info(outs[0])
        assert info["type"] == BF16 and info["dims"] == [m, n] and info["pointer"] != 0
        rc, raw = plugin.to_host(outs[0])
        plugin.ok(rc)
        direct = engine.execute(ex, [I.from_numpy(packed), I.from_numpy(scale, "bf16"), I.from_numpy(zero),
                                     I.from_numpy(g_idx), I.from_numpy(x, "bf16")])[0]
        assert raw == engine.to_host(direct)
        got = (np.frombuffer(raw, np.uint16).astype(np.uint32) << 16).view(np.float32).reshape(m, n)
        exact = x @ wref
        np.testing.assert_allclose(got, exact, rtol=2e-2, atol=1e-2 * np.abs(exact).max())
    finally:
        plugin.close()
