"""The device layer (include/ns.h) through the host wrappers: memory, queued copies, tickets, stamps, errors."""
import ctypes as C

import numpy as np
import pytest

from nextsycl_amd import Arena, DevBuf, Error, Gpu, HostBuf, api, gpus

pytestmark = pytest.mark.gpu


def test_enumeration(gpu):
    a = api()
    assert a.gpu_count() >= 1
    assert gpus()[0][0] == 0 and gpus()[0][1]
    units, mhz = gpu.units()
    assert units >= 64 and mhz > 500
    total, free = gpu.memory()
    assert total > (64 << 30) and free is not None and 0 < free <= total
    assert a.version().decode().startswith("nextsycl-amd")
    with pytest.raises(Error):
        Gpu.open(99)
    buf = C.create_string_buffer(8)
    assert a.gpu_name(99, buf, 8) == -1 and "no GPU 99" in a.error()


def test_copies_roundtrip(gpu):
    x = np.arange(1 << 18, dtype=np.uint32)
    b = DevBuf.of(gpu, x)
    assert np.array_equal(b.read(np.uint32), x)
    c = DevBuf(gpu, x.nbytes)
    a = gpu.api
    assert a.copy_dev(gpu.raw, c.ptr, b.ptr, x.nbytes) == 0
    assert np.array_equal(c.read(np.uint32), x)
    c.fill(0x7F)
    assert (c.read(np.uint8) == 0x7F).all()
    with pytest.raises(Error):
        b.read(np.uint8, count=x.nbytes + 1)
    v = b.view(1024, 4096)
    assert np.array_equal(v.read(np.uint32), x[256:256 + 1024])


@pytest.mark.parametrize("at,n", [(0, 1), (3, 77), (5, 3), (16, 4096), (1, 15), (15, 17), (7, 100001), (0, 1 << 20)])
def test_fill_any_alignment(gpu, at, n):
    """ns_fill is a kernel of the library's own (16-byte stores over the aligned body, byte stores over the ends): the
    span gets the value, the bytes either side keep theirs."""
    total = at + n + 37
    b = DevBuf(gpu, total)
    b.fill(0x11)
    a = gpu.api
    assert a.fill(gpu.raw, b.ptr + at, 0xAB, n) == 0
    got = b.read(np.uint8)
    assert (got[:at] == 0x11).all() and (got[at:at + n] == 0xAB).all() and (got[at + n:] == 0x11).all()


def test_copy_2d(gpu):
    a = gpu.api
    src = np.arange(32 * 64, dtype=np.uint8).reshape(32, 64)
    s, d = DevBuf.of(gpu, src), DevBuf(gpu, 32 * 48)
    d.fill(0)
    assert a.copy_2d(gpu.raw, d.ptr, 48, s.ptr + 8, 64, 40, 32) == 0
    got = d.read(np.uint8).reshape(32, 48)
    assert np.array_equal(got[:, :40], src[:, 8:48]) and (got[:, 40:] == 0).all()


def test_pinned_and_tickets(gpu):
    a = gpu.api
    n = 1 << 20
    h = HostBuf(gpu, n)
    h.array(np.uint8)[:] = 0x3C
    d = DevBuf(gpu, n)
    d.fill(0)
    t0, t1, t2 = C.c_int64(), C.c_int64(), C.c_int64()
    assert a.mark(gpu.raw, C.byref(t0)) == 0
    deps = (C.c_int64 * 1)(t0.value)
    assert a.stream_copy(gpu.raw, d.ptr, h.ptr, n, deps, 1, 0, C.byref(t1)) == 0
    assert a.await_(gpu.raw, t1.value) == 0
    assert (d.read(np.uint8) == 0x3C).all()
    assert a.stream_copy(gpu.raw, d.ptr, h.ptr, 0, None, 0, 1, C.byref(t2)) == 0
    assert t2.value == t1.value + 1


def test_stamps(gpu):
    d = DevBuf(gpu, 256 << 20)
    s0 = gpu.stamp()
    for _ in range(4):
        d.fill(1)
    s1 = gpu.stamp()
    ns = gpu.elapsed_ns(s0, s1)
    assert 1e4 < ns < 1e9
    bad = C.c_double()
    assert gpu.api.elapsed(gpu.raw, 60000, 60001, C.byref(bad)) == -1


def test_arena(gpu):
    ar = Arena(gpu, 1 << 20)
    a = ar.f32(1000)
    m = ar.mark()
    b = ar.bytes(5000)
    assert b.ptr >= a.ptr + 4000 and b.ptr % 256 == 0 and not b.owned
    ar.rewind(m)
    c = ar.bytes(100)
    assert c.ptr == b.ptr
    big = ar.bytes(2 << 20)
    assert big.owned and ar.spills == 1
    ar.reset()
    assert ar.bytes(16).ptr == a.ptr


def test_no_room_is_classified(gpu):
    assert Error("device allocation of 1024 bytes failed").is_no_room()
    assert Error.no_room("needs 2.0 GiB more").is_no_room()
    assert not Error("hip: hipStreamSynchronize: device lost").is_no_room()
    with pytest.raises(Error) as e:
        DevBuf(gpu, 1 << 46)
    assert e.value.is_no_room()
