"""GPU: the entry point that allocates nothing (axq_gemv_f32_static) against axq_gemv_f32.

Both run the same kernels (small-batch GEMV, 2..8 vectors per pass over the weights); the static entry point keeps
their scratch in a device array of the library instead of an allocation of the context.  Bar: bit-exact against the
existing entry point, which the parity tests hold to the oracle; the first case is also checked against the oracle
here.  The array is shared by every call on the GPU and keeps the last call's contents, so each case is run as two
calls in a row, the second with a smaller input (fewer vectors, a narrower weight).
"""
import numpy as np
import pytest

import oracle as o
from axonml_amd import quant as q
from axonml_amd._lib import MEM_DEVICE
from tests.util import MATMUL_RTOL, gen_weight, max_rel_err

pytestmark = pytest.mark.gpu


def _both(ctx, dw, x, bias):
    """(static entry point, existing entry point) on the same device buffers."""
    lib = ctx.lib
    batch, n = x.shape[0], dw.n_rows
    x_dev = ctx.to_device(x)
    b_dev = ctx.to_device(bias) if bias is not None else None
    y_dev = ctx.malloc(batch * n * 4)
    outs = []
    nan = np.full(batch * n, np.nan, np.float32)
    for call in (lambda: lib.axq_gemv_f32_static(ctx.handle, dw.handle, x_dev, batch, b_dev, y_dev),
                 lambda: lib.axq_gemv_f32(ctx.handle, dw.handle, x_dev, batch, b_dev, y_dev, MEM_DEVICE)):
        ctx.check(lib.axq_copy_to_device(ctx.handle, y_dev, nan.ctypes.data, nan.nbytes))
        ctx.check(call())
        ctx.synchronize()
        outs.append(ctx.to_host(y_dev, (batch, n), np.float32))
    ctx.free(x_dev)
    ctx.free(y_dev)
    if b_dev is not None:
        ctx.free(b_dev)
    return outs


@pytest.mark.parametrize("qtype", [o.Q4_K, o.Q4_0, o.Q4_1, o.Q8_0])
def test_static_entry_point_twice_in_a_row_second_call_smaller(ctx, qtype):
    rng = np.random.default_rng(70 + qtype)
    # first call: 8 vectors, k = 4096, few rows (K split over workgroups: partial sums in the scratch too)
    n1, k1 = 1024, 4096
    w1 = gen_weight(rng, n1, k1)
    p1 = o.quantize(qtype, w1)
    dw1 = q.DeviceWeight.upload(q.QuantizedTensor([n1, k1], qtype, p1), ctx)
    x1 = rng.standard_normal((8, k1)).astype(np.float32)
    bias1 = rng.standard_normal(n1).astype(np.float32)
    # second call: 3 vectors, k = 512: a smaller input that must not see what the first left behind
    n2, k2 = 160, 512
    p2 = o.quantize(qtype, gen_weight(rng, n2, k2))
    dw2 = q.DeviceWeight.upload(q.QuantizedTensor([n2, k2], qtype, p2), ctx)
    x2 = rng.standard_normal((3, k2)).astype(np.float32)

    lib = ctx.lib
    x1_dev, x2_dev, b1_dev = ctx.to_device(x1), ctx.to_device(x2), ctx.to_device(bias1)
    y1_dev, y2_dev = ctx.malloc(8 * n1 * 4), ctx.malloc(3 * n2 * 4)
    ctx.check(lib.axq_gemv_f32_static(ctx.handle, dw1.handle, x1_dev, 8, b1_dev, y1_dev))
    ctx.check(lib.axq_gemv_f32_static(ctx.handle, dw2.handle, x2_dev, 3, None, y2_dev))  # back to back, no sync between
    ctx.synchronize()
    got1 = ctx.to_host(y1_dev, (8, n1), np.float32)
    got2 = ctx.to_host(y2_dev, (3, n2), np.float32)
    for p in (x1_dev, x2_dev, b1_dev, y1_dev, y2_dev):
        ctx.free(p)

    static1, plain1 = _both(ctx, dw1, x1, bias1)
    static2, plain2 = _both(ctx, dw2, x2, None)
    assert np.array_equal(got1, plain1) and np.array_equal(static1, plain1)
    assert np.array_equal(got2, plain2) and np.array_equal(static2, plain2)
    # ... and the oracle's bar on both
    want1 = o.matmul_ref(qtype, p1, x1, n1, k1, bias1)
    want2 = o.matmul_ref(qtype, p2, x2, n2, k2)
    assert max_rel_err(got1, want1) <= MATMUL_RTOL
    assert max_rel_err(got2, want2) <= MATMUL_RTOL
    dw1.free()
    dw2.free()


def test_static_entry_point_at_the_decode_shapes(ctx):
    """Wide and narrow weights of the 7B layer (no K split / K split), 8 then 2 vectors."""
    rng = np.random.default_rng(5)
    for n, k, batch in ((14336, 4096, 8), (4096, 14336, 2)):
        p = o.quantize(o.Q4_K, gen_weight(rng, n, k, outlier_p=0.01))
        dw = q.DeviceWeight.upload(q.QuantizedTensor([n, k], o.Q4_K, p), ctx)
        x = rng.standard_normal((batch, k)).astype(np.float32)
        static, plain = _both(ctx, dw, x, None)
        assert np.array_equal(static, plain)
        assert max_rel_err(static, o.matmul_ref(o.Q4_K, p, x, n, k)) <= MATMUL_RTOL
        dw.free()


def test_static_entry_point_refuses_what_it_cannot_hold(ctx):
    lib = ctx.lib
    rng = np.random.default_rng(1)
    dummy = ctx.malloc(1 << 20)

    def call(dw, batch):
        return lib.axq_gemv_f32_static(ctx.handle, dw.handle, dummy, batch, None, dummy)

    ok = q.DeviceWeight.quantize(gen_weight(rng, 8, 512), q.QuantType.Q4_K, ctx)
    assert call(ok, 1) == -3 and call(ok, 9) == -3 and call(ok, 0) == -3          # AXQ_ERR_SHAPE_MISMATCH
    assert b"2..8" in lib.axq_last_error(ctx.handle)
    wide = q.DeviceWeight.quantize(gen_weight(rng, 2, 16384 + 256), q.QuantType.Q8_0, ctx)
    assert call(wide, 4) == -3
    assert b"static scratch" in lib.axq_last_error(ctx.handle)
    other = q.DeviceWeight.quantize(gen_weight(rng, 8, 512), q.QuantType.F16, ctx)  # not a block type
    assert call(other, 4) == -2                                                      # AXQ_ERR_INVALID_QUANT_TYPE
    ragged = q.DeviceWeight.quantize(gen_weight(rng, 8, 288), q.QuantType.Q8_0, ctx)
    assert call(ragged, 4) == -3                                                     # a shape limit: k % 256
    assert b"multiple of 256" in lib.axq_last_error(ctx.handle)
    assert lib.axq_gemv_f32_static(ctx.handle, ok.handle, None, 4, None, dummy) == -30  # AXQ_ERR_INVALID_ARGUMENT
    for w in (ok, wide, other, ragged):
        w.free()
    ctx.free(dummy)


def _hip():
    """The HIP runtime the library already has loaded, for the few calls the C ABI does not wrap (stream capture, memory info)."""
    import ctypes as C

    hip = C.CDLL("libamdhip64.so")
    vp = C.c_void_p
    hip.hipStreamCreateWithFlags.argtypes = [C.POINTER(vp), C.c_uint]
    hip.hipStreamDestroy.argtypes = [vp]
    hip.hipStreamSynchronize.argtypes = [vp]
    hip.hipStreamBeginCapture.argtypes = [vp, C.c_int]
    hip.hipStreamEndCapture.argtypes = [vp, C.POINTER(vp)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(vp), vp, C.POINTER(vp), C.c_char_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [vp, vp]
    hip.hipGraphExecDestroy.argtypes = [vp]
    hip.hipGraphDestroy.argtypes = [vp]
    hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    return hip


def test_static_entry_point_under_stream_capture_and_with_no_change_in_free_memory(ctx):
    """What the entry point is for: two calls recorded into a HIP graph (global capture mode refuses every allocation
    made meanwhile, so a hidden hipMalloc would fail the capture), replayed three times with eager work and
    synchronisations between the replays, every replay equal to the eager result; and the device's free memory is the
    same before and after a run of plain calls."""
    import ctypes as C

    hip, lib = _hip(), ctx.lib
    rng = np.random.default_rng(17)
    n1, k1, n2, k2 = 4096, 4096, 512, 1024   # the first call splits K over workgroups (partial sums in the scratch)
    p1 = o.quantize(o.Q4_K, gen_weight(rng, n1, k1))
    p2 = o.quantize(o.Q4_0, gen_weight(rng, n2, k2))
    dw1 = q.DeviceWeight.upload(q.QuantizedTensor([n1, k1], o.Q4_K, p1), ctx)
    dw2 = q.DeviceWeight.upload(q.QuantizedTensor([n2, k2], o.Q4_0, p2), ctx)
    x1, x2 = rng.standard_normal((8, k1)).astype(np.float32), rng.standard_normal((3, k2)).astype(np.float32)
    x1_dev, x2_dev = ctx.to_device(x1), ctx.to_device(x2)
    y1_dev, y2_dev = ctx.malloc(8 * n1 * 4), ctx.malloc(3 * n2 * 4)

    def run_eager():
        ctx.check(lib.axq_gemv_f32_static(ctx.handle, dw1.handle, x1_dev, 8, None, y1_dev))
        ctx.check(lib.axq_gemv_f32_static(ctx.handle, dw2.handle, x2_dev, 3, None, y2_dev))
        ctx.synchronize()
        return ctx.to_host(y1_dev, (8, n1), np.float32), ctx.to_host(y2_dev, (3, n2), np.float32)

    want1, want2 = run_eager()   # also the first use of both kernels on this device, outside any capture
    assert max_rel_err(want1, o.matmul_ref(o.Q4_K, p1, x1, n1, k1)) <= MATMUL_RTOL
    assert max_rel_err(want2, o.matmul_ref(o.Q4_0, p2, x2, n2, k2)) <= MATMUL_RTOL

    # free memory across plain calls
    free0, free1, total = C.c_size_t(), C.c_size_t(), C.c_size_t()
    assert hip.hipMemGetInfo(C.byref(free0), C.byref(total)) == 0
    for _ in range(20):
        ctx.check(lib.axq_gemv_f32_static(ctx.handle, dw1.handle, x1_dev, 8, None, y1_dev))
        ctx.check(lib.axq_gemv_f32_static(ctx.handle, dw2.handle, x2_dev, 3, None, y2_dev))
    ctx.synchronize()
    assert hip.hipMemGetInfo(C.byref(free1), C.byref(total)) == 0
    assert free1.value == free0.value

    # the same two calls as a graph on a stream of the caller's
    stream, graph, gexec = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert hip.hipStreamCreateWithFlags(C.byref(stream), 1) == 0   # hipStreamNonBlocking
    ctx.check(lib.axq_set_stream(ctx.handle, stream))
    nan1, nan2 = np.full(8 * n1, np.nan, np.float32), np.full(3 * n2, np.nan, np.float32)
    try:
        assert hip.hipStreamBeginCapture(stream, 0) == 0           # hipStreamCaptureModeGlobal
        st1 = lib.axq_gemv_f32_static(ctx.handle, dw1.handle, x1_dev, 8, None, y1_dev)
        st2 = lib.axq_gemv_f32_static(ctx.handle, dw2.handle, x2_dev, 3, None, y2_dev)
        assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert st1 == 0 and st2 == 0
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        for _ in range(3):
            ctx.check(lib.axq_copy_to_device(ctx.handle, y1_dev, nan1.ctypes.data, nan1.nbytes))   # eager work between replays
            ctx.check(lib.axq_copy_to_device(ctx.handle, y2_dev, nan2.ctypes.data, nan2.nbytes))
            assert hip.hipGraphLaunch(gexec, stream) == 0
            assert hip.hipStreamSynchronize(stream) == 0
            assert np.array_equal(ctx.to_host(y1_dev, (8, n1), np.float32), want1)
            assert np.array_equal(ctx.to_host(y2_dev, (3, n2), np.float32), want2)
    finally:
        ctx.check(lib.axq_set_stream(ctx.handle, None))
        if gexec:
            hip.hipGraphExecDestroy(gexec)
        if graph:
            hip.hipGraphDestroy(graph)
        hip.hipStreamDestroy(stream)
    for p in (x1_dev, x2_dev, y1_dev, y2_dev):
        ctx.free(p)
    dw1.free()
    dw2.free()
