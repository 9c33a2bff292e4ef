"""The checked layer over the library: GPUs, device and pinned host buffers that free themselves, copies with their
sizes checked, a bump arena for per-pass scratch. Mirrors crates/core/src/lib.rs:17-60,133-503 - same ownership rules:
the caller (an engine) owns all device memory, kernels never allocate, an arena's views are valid until it is rewound
(legal because the GPU's queue is in order)."""
import ctypes as C
import threading

import numpy as np

from .sys import Api

NO_ROOM = "no room: "


class Error(Exception):
    """A failed call: "<what>: <the library's reason>" (crates/core/src/lib.rs:17-44)."""

    @staticmethod
    def no_room(msg):
        return Error(NO_ROOM + str(msg))

    def is_no_room(self):
        """No room now - retryable: Error.no_room, a failed device allocation, or the runtime out of device memory."""
        s = str(self)
        return s.startswith(NO_ROOM) or ("device allocation of " in s and " bytes failed" in s) or "OUT_OF_DEVICE_MEMORY" in s or \
            "hipErrorOutOfMemory" in s or "out of memory" in s


_api = None
_api_lock = threading.Lock()


def api():
    """The kernel library, loaded once."""
    global _api
    with _api_lock:
        if _api is None:
            _api = Api()
    return _api


def check(a, rc, what):
    if rc != 0:
        raise Error("%s: %s" % (what, a.error()))


def gpus():
    """[(index, name)] in the order Gpu.open takes."""
    a = api()
    out = []
    for i in range(a.gpu_count()):
        buf = C.create_string_buffer(256)
        check(a, a.gpu_name(i, buf, 256), "naming GPU %d" % i)
        out.append((i, buf.value.decode()))
    return out


class Gpu:
    """One GPU with its in-order queue."""

    def __init__(self, index=0):
        a = api()
        n = a.gpu_count()
        if index < 0 or index >= n:
            raise Error("no GPU %d (%d found)" % (index, n))
        self.api, self.index = a, index
        raw = C.c_void_p()
        check(a, a.gpu_open(index, C.byref(raw)), "opening GPU %d" % index)
        self.raw = raw
        buf = C.create_string_buffer(256)
        a.gpu_name(index, buf, 256)
        self.name = buf.value.decode()
        pci = C.create_string_buffer(64)
        self.pci = pci.value.decode() if a.gpu_pci(index, pci, 64) == 0 and pci.value else None

    @staticmethod
    def open(index=0):
        return Gpu(index)

    def close(self):
        if self.raw:
            self.api.sync(self.raw)
            self.api.gpu_close(self.raw)
            self.raw = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def units(self):
        u, m = C.c_int(), C.c_int()
        check(self.api, self.api.gpu_units(self.index, C.byref(u), C.byref(m)), "the GPU's units")
        return u.value, m.value

    def memory(self):
        t, f = C.c_uint64(), C.c_int64()
        check(self.api, self.api.gpu_memory(self.raw, C.byref(t), C.byref(f)), "the GPU's memory")
        return t.value, (f.value if f.value >= 0 else None)

    def sync(self):
        check(self.api, self.api.sync(self.raw), "waiting for the GPU")

    def stamp(self):
        t = C.c_int64()
        check(self.api, self.api.stamp(self.raw, C.byref(t)), "a stamp")
        return t.value

    def elapsed_ns(self, t0, t1):
        ns = C.c_double()
        check(self.api, self.api.elapsed(self.raw, t0, t1, C.byref(ns)), "the time between two stamps")
        return ns.value


class DevBuf:
    """Device memory of one GPU; a view (`view`, an Arena's) does not own its memory."""

    def __init__(self, gpu, nbytes, _ptr=None, _owner=None):
        self.gpu, self.len = gpu, int(nbytes)
        if _ptr is None:
            p = C.c_void_p()
            check(gpu.api, gpu.api.alloc(gpu.raw, max(self.len, 1), C.byref(p)), "allocating %d bytes on %s" % (self.len, gpu.name))
            self.ptr, self.owned, self._owner = p.value, True, None
        else:
            self.ptr, self.owned, self._owner = _ptr, False, _owner

    def __del__(self):
        try:
            if self.owned and self.ptr and self.gpu.raw:
                self.gpu.api.free(self.gpu.raw, self.ptr)
                self.ptr = None
        except Exception:
            pass

    def bounds(self, at, n):
        if at < 0 or n < 0 or at + n > self.len:
            raise Error("bytes %d..%d of a %d-byte buffer" % (at, at + n, self.len))

    def view(self, at, n):
        self.bounds(at, n)
        return DevBuf(self.gpu, n, _ptr=self.ptr + at, _owner=self)

    def write(self, src, at=0):
        """Host array into [at, at + bytes), waiting (so the source may be a temporary)."""
        src = np.ascontiguousarray(src)
        self.bounds(at, src.nbytes)
        g = self.gpu
        check(g.api, g.api.copy_to(g.raw, self.ptr + at, src.ctypes.data, src.nbytes), "copying to the GPU")
        g.sync()

    def read(self, dtype, count=None, at=0):
        """[at, ...) as a host array of `dtype`, waiting."""
        dt = np.dtype(dtype)
        n = (self.len - at) // dt.itemsize if count is None else int(count)
        out = np.empty(n, dt)
        self.bounds(at, out.nbytes)
        g = self.gpu
        check(g.api, g.api.copy_from(g.raw, out.ctypes.data, self.ptr + at, out.nbytes), "copying from the GPU")
        g.sync()
        return out

    def fill(self, v=0):
        g = self.gpu
        check(g.api, g.api.fill(g.raw, self.ptr, v, self.len), "filling")

    @staticmethod
    def of(gpu, arr):
        """A new buffer holding the host array."""
        arr = np.ascontiguousarray(arr)
        b = DevBuf(gpu, arr.nbytes)
        b.write(arr)
        return b


class HostBuf:
    """Pinned host memory: the fast side of a GPU's copies."""

    def __init__(self, gpu, nbytes):
        self.gpu, self.len = gpu, int(nbytes)
        p = C.c_void_p()
        check(gpu.api, gpu.api.alloc_host(gpu.raw, max(self.len, 1), C.byref(p)), "pinning %d bytes" % self.len)
        self.ptr = p.value

    def array(self, dtype):
        dt = np.dtype(dtype)
        return np.ctypeslib.as_array((C.c_uint8 * self.len).from_address(self.ptr)).view(dt)

    def __del__(self):
        try:
            if self.ptr and self.gpu.raw:
                self.gpu.api.free_host(self.gpu.raw, self.ptr)
                self.ptr = None
        except Exception:
            pass


class Arena:
    """A bump allocator over one device allocation: a pass's temporaries (attention scratch) without an allocation
    each. Requests that do not fit get an allocation of their own (counted in `spills`)."""

    def __init__(self, gpu, nbytes):
        self.buf = DevBuf(gpu, nbytes)
        self.off = self.peak = self.spills = 0

    def bytes(self, n):
        at = (self.off + 255) // 256 * 256
        if at + n > self.buf.len:
            self.spills += 1
            return DevBuf(self.buf.gpu, n)
        self.off = at + n
        self.peak = max(self.peak, self.off)
        return self.buf.view(at, max(n, 1) if at + max(n, 1) <= self.buf.len else n)

    def f32(self, n):
        return self.bytes(4 * n)

    def reset(self):
        self.off = 0

    def mark(self):
        return self.off

    def rewind(self, mark):
        if mark < self.off:
            self.off = mark
