"""The configs[1] chain captured into a HIP graph through the library's own stream and replayed.

A caller that wants the three launches of the chain without their launch gaps can capture them: the entry points of
the path queue kernels on the context's stream and nothing else (no allocation, no memset, no synchronization; the
one block of device memory the library owns, the result tables of the 16-bit unary operations, is allocated and
filled when the context is created), and hmr_ext_stream hands the stream out. The test captures one pass of the chain (after a pass that warms the host
layer's allocator, so that the capture finds its buffers in the cache), replays it several times with eager work and
synchronizations of its own between the replays, and compares every replay with the eager result, bit for bit."""
import ctypes

import numpy as np
import pytest

from homura_amd import capi
from tests import oracle
from tests.support import DT, GPU, bits, from_f64, h, normal, tensor, uniform

pytestmark = pytest.mark.gpu
h.register_cpu_backend(oracle.backend_address())

RELAXED = 2  # hipStreamCaptureModeRelaxed


def test_the_chain_replays_from_a_graph_with_the_eager_bits():
    hip = ctypes.CDLL("libamdhip64.so")
    stream = ctypes.c_void_p(h.stream_handle(GPU))
    B, S, H = 4, 512, 1024
    n = B * S * H
    x = tensor(from_f64(normal(11, n), DT.BF16), DT.BF16, [B, S, H], GPU)
    bias = tensor(from_f64(normal(12, H, 0.0, 0.02), DT.BF16), DT.BF16, [H], GPU)
    scale = tensor(from_f64(uniform(13, B * S, 0.5, 1.5), DT.BF16), DT.BF16, [B, S, 1], GPU)
    residual = tensor(normal(14, n).astype(np.float32), DT.F32, [B, S, H], GPU)

    def chain():
        return x.add(bias).mul(scale).add(residual)

    eager = bits(chain())   # also leaves the chain's buffers in the allocator's cache
    h.synchronize(GPU)
    graph, executable = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamBeginCapture(stream, RELAXED) == 0
    try:
        # The intermediates stay referenced for as long as the graph lives: a replay writes them again, so their
        # buffers must not go back to the allocator's cache.
        t = x.add(bias)
        u = t.mul(scale)
        out = u.add(residual)
    finally:
        status = hip.hipStreamEndCapture(stream, ctypes.byref(graph))
    assert status == 0 and graph.value
    assert hip.hipGraphInstantiate(ctypes.byref(executable), graph, None, None, ctypes.c_size_t(0)) == 0
    try:
        # Nothing ran during the capture: the result buffer still holds what an earlier pass left there or nothing
        # in particular. Overwrite it, so that only a replay can make it right.
        out.fill_(0.0)
        for replay in range(4):
            assert hip.hipGraphLaunch(executable, stream) == 0
            h.synchronize(GPU)
            assert np.array_equal(bits(out), eager), f"replay {replay}"
            # Eager work of the program between replays, on the same stream, taking buffers from the same cache.
            other = x.mul(scale).add(bias)
            assert np.array_equal(bits(chain()), eager), f"eager pass after replay {replay}"
            out.fill_(float(replay))
            del other
            h.synchronize(GPU)
    finally:
        hip.hipGraphExecDestroy(executable)
        hip.hipGraphDestroy(graph)
        del t, u


def test_the_first_table_lookup_of_a_context_may_be_captured():
    """A fresh context whose FIRST 16-bit unary operation of table size is queued while its stream is capturing:
    the capture records the lookup only (the tables exist since the context was created), an eager call of the
    same operation before any replay has the oracle's bits, and so has every replay."""
    hip = ctypes.CDLL("libamdhip64.so")
    patterns = np.arange(1 << 16, dtype=np.uint16)
    expected = bits(tensor(patterns, DT.BF16, [1 << 16]).silu())
    ctx = capi.Context(0)
    try:
        stream = ctypes.c_void_p(ctx.stream())
        src = ctx.upload(patterns)
        captured, eager = ctx.malloc(patterns.nbytes), ctx.malloc(patterns.nbytes)
        for buf in (captured, eager):
            capi.check(capi.lib.hmr_memset(ctx.handle, buf.ptr, 0xA5, patterns.nbytes))
        ctx.synchronize()
        d_src = capi.make_desc(src.ptr, capi.BF16, [1 << 16], [1])
        d_cap = capi.make_desc(captured.ptr, capi.BF16, [1 << 16], [1])
        d_eager = capi.make_desc(eager.ptr, capi.BF16, [1 << 16], [1])
        graph, executable = ctypes.c_void_p(), ctypes.c_void_p()
        assert hip.hipStreamBeginCapture(stream, 0) == 0  # hipStreamCaptureModeGlobal: an allocation would fail it
        try:
            status = capi.lib.hmr_unary(ctx.handle, capi.UNARY["silu"], ctypes.byref(d_cap), ctypes.byref(d_src))
        finally:
            ended = hip.hipStreamEndCapture(stream, ctypes.byref(graph))
        assert status == 0 and ended == 0 and graph.value
        assert hip.hipGraphInstantiate(ctypes.byref(executable), graph, None, None, ctypes.c_size_t(0)) == 0
        try:
            capi.check(capi.lib.hmr_unary(ctx.handle, capi.UNARY["silu"], ctypes.byref(d_eager), ctypes.byref(d_src)))
            ctx.synchronize()
            assert np.array_equal(eager.download(np.uint16, 1 << 16), expected), "eager lookup before any replay"
            assert np.all(captured.download(np.uint16, 1 << 16) == 0xA5A5), "the capture ran nothing"
            for replay in range(3):
                assert hip.hipGraphLaunch(executable, stream) == 0
                ctx.synchronize()
                assert np.array_equal(captured.download(np.uint16, 1 << 16), expected), f"replay {replay}"
                capi.check(capi.lib.hmr_memset(ctx.handle, captured.ptr, replay, patterns.nbytes))
                ctx.synchronize()
        finally:
            hip.hipGraphExecDestroy(executable)
            hip.hipGraphDestroy(graph)
        for buf in (src, captured, eager):
            buf.free()
    finally:
        ctx.close()
