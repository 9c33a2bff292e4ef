"""ns_attn_decode_static - the decode entry point that allocates nothing (its partials live in an array inside the
library's code object) - against ns_attn_decode_t on the same inputs: the same kernels, so the same bits. Two calls in a
row share the array; the second, smaller one must not see anything of the first."""
import numpy as np
import pytest

from helpers import gpu_decode, make_kv, make_q
from nextsycl_amd import DevBuf
from nextsycl_amd.attn import BF16, F16, F32
from nextsycl_amd.core import Error

pytestmark = pytest.mark.gpu


def _static(ops, qt, kt, qd, bufs, T, Hq, Hkv, D, cap, p0, win=0):
    g = ops.gpu
    ob = DevBuf(g, T * Hq * D * (4 if qt == F32 else 2))
    ob.fill(0xFF)
    ops.decode_static(qt, kt, DevBuf.of(g, qd), Hq * D, bufs[0], bufs[1], T, Hq, Hkv, D, cap, p0, ob, win=win)
    return ob.read(np.float32 if qt == F32 else np.uint16)


def test_static_scratch_decode_matches_the_buffer_form(ops):
    g = ops.gpu
    # a large pass first (many splits, 4 rows), then smaller ones of other shapes: each against ns_attn_decode_t's bits
    shapes = [(4, 32, 4, 128, 30000, 0, 0, F16), (1, 8, 2, 128, 700, 0, 0, F32), (2, 16, 2, 256, 2500, 0, 1, F32), (3, 16, 4, 128, 5000, 1024, 3, BF16),
              (1, 32, 8, 128, 129, 0, 2, F16)]
    for rep in range(2):
        for i, (T, Hq, Hkv, D, p0, win, kt, qt) in enumerate(shapes):
            cap = p0 + T
            kc, vc = make_kv(kt, Hkv, D, cap, cap, cfg=i)
            qd, _ = make_q(qt, T, Hq, D, cfg=i)
            bufs = (DevBuf.of(g, kc), DevBuf.of(g, vc))
            _, want = gpu_decode(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win, bufs=bufs)
            got = _static(ops, qt, kt, qd, bufs, T, Hq, Hkv, D, cap, p0, win=win)
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (rep, i)


def test_static_scratch_decode_rejects_what_does_not_fit(ops):
    g = ops.gpu
    b = DevBuf(g, 1 << 16)
    # 16 rows x 64 heads over 128 splits: 68 MB of partials against the array's 16 MiB - refused before any launch
    T, Hq, Hkv, D, p0 = 16, 64, 4, 128, 200000
    assert ops.k.attn_decode_scratch(T, Hq, Hkv, D, p0, 0) > (4 << 20)
    rc = ops.k.attn_decode_static(g.raw, 0, 0, 0, b.ptr, Hq * D, b.ptr, b.ptr, T, Hq, Hkv, D, p0 + T, p0, 0, 0.0, b.ptr)
    assert rc == -1 and "the array holds" in ops.k.api.error()
    with pytest.raises(Error):
        ops.decode_static(F32, 0, b, Hq * D, b, b, 17, Hq, Hkv, D, 64, 0, b)


def test_static_scratch_decode_allocates_nothing(ops):
    """A run of calls leaves the device's free memory where it was (ns_gpu_memory around 50 calls whose buffers all exist
    beforehand), and a call goes through a stream capture that forbids allocation (mode "global": any hipMalloc on any
    thread fails the capture) - kernel launches are all it queues."""
    import ctypes as C

    g = ops.gpu
    T, Hq, Hkv, D, p0 = 2, 16, 2, 128, 3000
    cap = p0 + T
    kc, vc = make_kv(0, Hkv, D, cap, cap)
    qd, _ = make_q(F16, T, Hq, D)
    kcb, vcb, qb, ob = DevBuf.of(g, kc), DevBuf.of(g, vc), DevBuf.of(g, qd), DevBuf(g, T * Hq * D * 2)
    ops.decode_static(F16, 0, qb, Hq * D, kcb, vcb, T, Hq, Hkv, D, cap, p0, ob)      # (first call: anything lazy has happened)
    g.sync()
    want = ob.read(np.uint16)
    total, free0 = C.c_uint64(), C.c_int64()
    assert g.api.gpu_memory(g.raw, C.byref(total), C.byref(free0)) == 0
    for _ in range(50):
        ops.decode_static(F16, 0, qb, Hq * D, kcb, vcb, T, Hq, Hkv, D, cap, p0, ob)
    g.sync()
    free1 = C.c_int64()
    assert g.api.gpu_memory(g.raw, C.byref(total), C.byref(free1)) == 0
    assert free1.value == free0.value
    # under a capture that refuses allocation
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    stream = C.cast(C.c_void_p(g.api.gpu_queue(g.raw)), C.POINTER(C.c_void_p))[0]
    graph, ex = C.c_void_p(), C.c_void_p()
    ob.fill(0)
    g.sync()
    assert hip.hipStreamBeginCapture(stream, 0) == 0                                   # hipStreamCaptureModeGlobal
    try:
        ops.decode_static(F16, 0, qb, Hq * D, kcb, vcb, T, Hq, Hkv, D, cap, p0, ob)
    finally:
        rc = hip.hipStreamEndCapture(stream, C.byref(graph))
    assert rc == 0 and graph.value
    assert hip.hipGraphInstantiate(C.byref(ex), graph, None, None, 0) == 0
    try:
        assert hip.hipGraphLaunch(ex, stream) == 0
        g.sync()
        assert np.array_equal(ob.read(np.uint16), want)
    finally:
        hip.hipGraphExecDestroy(ex)
        hip.hipGraphDestroy(graph)
