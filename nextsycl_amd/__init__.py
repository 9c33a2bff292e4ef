"""nextsycl_amd: the host side of libnextsycl-llm.so - nextsycl's LLM attention path as hand-written gfx950 HIP kernels
behind the reference's own C ABI.

    sys.py    the library opened at run time, its ns.h symbols bound by name      (reference: crates/sys/src/lib.rs)
    core.py   Gpu / DevBuf / HostBuf / Arena: memory that frees itself, checked copies  (reference: crates/core/src/lib.rs)
    attn.py   the attention ABI bound by name + size-checked wrappers              (reference: llm/<arch>/src/ffi.rs, ops.rs)
    build.py  hipcc recipe for the in-tree library

The compute path is the HIP library only: nothing here falls back to a CPU or PyTorch implementation, and loading
fails loudly when the library is missing."""
from .core import Arena, DevBuf, Error, Gpu, HostBuf, api, gpus  # noqa: F401
from .sys import Api, library_path  # noqa: F401
