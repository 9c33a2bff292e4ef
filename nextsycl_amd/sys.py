"""Raw bindings to libnextsycl-llm.so: one ctypes function per declaration of include/ns.h, the library opened at run
time (dlopen), not linked - the host side imports anywhere, and a missing or stale library fails at load, loudly.
An engine-side table binds its own kernels by name through `Api.symbol`. Mirrors crates/sys/src/lib.rs:26-60,138-299."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libnextsycl-llm.so"

i32, i64, u64, f32, f64 = C.c_int, C.c_int64, C.c_uint64, C.c_float, C.c_double
P, SZ, STR = C.c_void_p, C.c_size_t, C.c_char_p

# name -> (restype, argtypes): include/ns.h in declaration order
NS_H = {
    "ns_last_error": (STR, []),
    "ns_version": (STR, []),
    "ns_gpu_count": (i32, []),
    "ns_gpu_name": (i32, [i32, P, SZ]),
    "ns_gpu_pci": (i32, [i32, P, SZ]),
    "ns_gpu_units": (i32, [i32, C.POINTER(i32), C.POINTER(i32)]),
    "ns_gpu_open": (i32, [i32, C.POINTER(P)]),
    "ns_gpu_close": (None, [P]),
    "ns_gpu_queue": (P, [P]),
    "ns_gpu_memory": (i32, [P, C.POINTER(u64), C.POINTER(i64)]),
    "ns_alloc": (i32, [P, SZ, C.POINTER(P)]),
    "ns_free": (i32, [P, P]),
    "ns_alloc_host": (i32, [P, SZ, C.POINTER(P)]),
    "ns_free_host": (i32, [P, P]),
    "ns_copy_to": (i32, [P, P, P, SZ]),
    "ns_copy_from": (i32, [P, P, P, SZ]),
    "ns_copy_dev": (i32, [P, P, P, SZ]),
    "ns_copy_2d": (i32, [P, P, SZ, P, SZ, SZ, SZ]),
    "ns_mark": (i32, [P, C.POINTER(i64)]),
    "ns_stream_copy": (i32, [P, P, P, SZ, C.POINTER(i64), i32, i32, C.POINTER(i64)]),
    "ns_await": (i32, [P, i64]),
    "ns_stamp": (i32, [P, C.POINTER(i64)]),
    "ns_elapsed": (i32, [P, i64, i64, C.POINTER(f64)]),
    "ns_fill": (i32, [P, P, C.c_uint8, SZ]),
    "ns_sync": (i32, [P]),
    "ns_copy_peer": (i32, [P, P, P, P, SZ, P]),
}
# a library built before it lacks this one; everything else must be there (crates/sys/src/lib.rs:204-235)
OPTIONAL = {"ns_copy_2d"}


def library_path():
    """NEXTSYCL_LIB, else the in-tree build (nextsycl_amd/lib/)."""
    return os.environ.get("NEXTSYCL_LIB") or os.path.join(HERE, "lib", LIB_NAME)


class Api:
    """The opened library: its ns.h functions as attributes without the ns_ prefix (`api.gpu_open`, `api.sync`...)."""

    def __init__(self, path=None):
        self.path = path or library_path()
        if not os.path.exists(self.path):
            raise OSError("%s not found: build it with `python -m nextsycl_amd.build` (hipcc, gfx950)" % self.path)
        # RTLD_GLOBAL as the reference opens a kind's library: a later library resolves ns_fail from it
        self.handle = C.CDLL(self.path, mode=C.RTLD_GLOBAL)
        for name, (res, args) in NS_H.items():
            try:
                fn = getattr(self.handle, name)
            except AttributeError:
                if name in OPTIONAL:
                    setattr(self, name[3:], None)
                    continue
                raise OSError("%s: missing symbol %s" % (self.path, name))
            fn.restype, fn.argtypes = res, args
            # `await` is a keyword: bound as await_, as the reference's table names it (crates/sys/src/lib.rs:54)
            setattr(self, "await_" if name == "ns_await" else name[3:], fn)

    def symbol(self, name, restype, argtypes):
        """An engine's own entry point by name; a missing one is a load error (llm/qwen35/src/ffi.rs:139-145)."""
        try:
            fn = getattr(self.handle, name)
        except AttributeError:
            raise OSError("%s: missing symbol %s" % (self.path, name))
        fn.restype, fn.argtypes = restype, argtypes
        return fn

    def error(self):
        e = self.last_error()
        return e.decode("utf-8", "replace") if e else ""
