"""A decode token's attention - the KV store of the token's row and ns_attn_decode_static over the cache - captured into a
HIP graph on the library's stream and replayed: what a serving loop that cannot allocate (and does not want a launch's
host cost a kernel) does with these entry points. Every replay, with eager copies and synchronizations between them, is
held to the bits of the same two calls made eagerly. The graph holds kernel launches only (the library records no memset
and no allocation)."""
import ctypes as C

import numpy as np
import pytest

from helpers import make_kv, make_q
from nextsycl_amd import DevBuf, Gpu
from nextsycl_amd.attn import F16, Ops
from oracle import orc

pytestmark = pytest.mark.gpu


def _hip():
    h = C.CDLL("libamdhip64.so")
    h.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    h.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    h.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_char_p, C.c_size_t]
    h.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    h.hipGraphExecDestroy.argtypes = [C.c_void_p]
    h.hipGraphDestroy.argtypes = [C.c_void_p]
    h.hipStreamSynchronize.argtypes = [C.c_void_p]
    return h


def test_decode_token_in_a_graph():
    hip = _hip()
    g = Gpu.open(0)                                  # a handle (and stream) of its own: a capture gone wrong stays here
    ops = Ops(g)
    T, Hq, Hkv, D, p0, kt, qt = 1, 32, 8, 128, 5000, 0, F16
    cap = p0 + T
    kc, vc = make_kv(kt, Hkv, D, cap, p0)            # the context; the token's own row is stored by the graph
    kcb, vcb = DevBuf.of(g, kc), DevBuf.of(g, vc)
    kb, vb = DevBuf(g, Hkv * D * 4), DevBuf(g, Hkv * D * 4)
    qb, ob = DevBuf(g, Hq * D * 2), DevBuf(g, Hq * D * 2)
    stream = C.cast(C.c_void_p(g.api.gpu_queue(g.raw)), C.POINTER(C.c_void_p))[0]

    def token():
        ops.kv_store(kt, kb, Hkv * D, vb, Hkv * D, T, Hkv, D, cap, p0, kcb, vcb)
        ops.decode_static(qt, kt, qb, Hq * D, kcb, vcb, T, Hq, Hkv, D, cap, p0, ob)

    g.sync()
    graph, ex = C.c_void_p(), C.c_void_p()
    assert hip.hipStreamBeginCapture(stream, 2) == 0                 # hipStreamCaptureModeRelaxed
    try:
        token()
    finally:
        rc = hip.hipStreamEndCapture(stream, C.byref(graph))
    assert rc == 0 and graph.value
    assert hip.hipGraphInstantiate(C.byref(ex), graph, None, None, 0) == 0
    try:
        for rep in range(3):
            k, v = orc.randn(70 + rep, (T, Hkv * D)), orc.randn(80 + rep, (T, Hkv * D))
            qd, _ = make_q(qt, T, Hq, D, cfg=rep)
            kb.write(k)
            vb.write(v)
            qb.write(qd)
            ob.fill(0xFF)
            g.sync()
            assert hip.hipGraphLaunch(ex, stream) == 0
            assert hip.hipStreamSynchronize(stream) == 0
            got = ob.read(np.uint16)
            row_k = kcb.read(np.uint8).reshape(kc.shape)[:, p0].copy()
            ob.fill(0xFF)
            token()                                                  # the same two calls, eagerly
            want = ob.read(np.uint16)
            assert np.array_equal(got, want), rep
            assert np.array_equal(row_k, orc.kv_store(kt, k, v, Hkv, D, T, 0)[0][:, 0]), rep      # the token's row went in
    finally:
        hip.hipGraphExecDestroy(ex)
        hip.hipGraphDestroy(graph)
        g.close()


def test_decode_token_through_the_library_graph_calls():
    """The same token recorded and replayed through ns_q35_graph_begin / _end / _launch / _free (the reference's four
    calls, here over HIP stream capture): nothing runs while recording, every replay equals the eager calls bit for bit,
    a graph still recording cannot be launched, and one freed while recording leaves the stream usable."""
    g = Gpu.open(0)
    ops = Ops(g)
    T, Hq, Hkv, D, p0, kt, qt = 2, 16, 2, 128, 3000, 0, F16
    cap = p0 + T
    kc, vc = make_kv(kt, Hkv, D, cap, p0)
    kcb, vcb = DevBuf.of(g, kc), DevBuf.of(g, vc)
    kb, vb = DevBuf(g, T * Hkv * D * 4), DevBuf(g, T * Hkv * D * 4)
    qb, ob = DevBuf(g, T * Hq * D * 2), DevBuf(g, T * Hq * D * 2)

    def token():
        ops.kv_store(kt, kb, Hkv * D, vb, Hkv * D, T, Hkv, D, cap, p0, kcb, vcb)
        ops.decode_static(qt, kt, qb, Hq * D, kcb, vcb, T, Hq, Hkv, D, cap, p0, ob)

    try:
        # a recording that is dropped: freed before it ended
        h = C.c_void_p()
        ops.ok(ops.k.q35_graph_begin(ops.raw(), C.byref(h)), "graph begin")
        token()
        assert ops.k.q35_graph_launch(ops.raw(), h) == -1 and "not finished" in g.api.error()
        # while the stream records, calls that would wait for it are refused (and the recording survives them), and a
        # second recording cannot begin
        assert g.api.sync(g.raw) == -1 and "recording" in g.api.error()
        h2 = C.c_void_p()
        assert ops.k.q35_graph_begin(ops.raw(), C.byref(h2)) == -1 and "recording" in g.api.error()
        ops.k.q35_graph_free(h)
        g.sync()                                        # (the stream runs again)
        g.sync()
        # the recording that is kept
        ob.fill(0xFF)
        g.sync()
        h = C.c_void_p()
        ops.ok(ops.k.q35_graph_begin(ops.raw(), C.byref(h)), "graph begin")
        try:
            token()
        finally:
            ops.ok(ops.k.q35_graph_end(ops.raw(), h), "graph end")
        g.sync()
        assert (ob.read(np.uint16) == 0xFFFF).all()                  # recorded, not run
        for rep in range(3):
            k, v = orc.randn(170 + rep, (T, Hkv * D)), orc.randn(180 + rep, (T, Hkv * D))
            qd, _ = make_q(qt, T, Hq, D, cfg=rep)
            kb.write(k)
            vb.write(v)
            qb.write(qd)
            ob.fill(0xFF)
            g.sync()
            ops.ok(ops.k.q35_graph_launch(ops.raw(), h), "graph launch")
            g.sync()
            got = ob.read(np.uint16)
            ob.fill(0xFF)
            token()
            assert np.array_equal(got, ob.read(np.uint16)), rep
        ops.k.q35_graph_free(h)
    finally:
        g.close()
