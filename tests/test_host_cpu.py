"""What needs no GPU: the library loads and exports every symbol the headers declare, the host wrappers' own logic
(row sizes, error classification, scratch sizing through the C ABI's pure functions)."""
import ctypes as C
import os
import re

import pytest

from nextsycl_amd import Error, library_path
from nextsycl_amd.attn import ATTN_H, MLA_H, PRE_H, kv_row_bytes
from nextsycl_amd.sys import NS_H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def handle():
    if not os.path.exists(library_path()):
        from nextsycl_amd.build import build
        build()
    return C.CDLL(library_path())


def _declared(header):
    """extern "C" function names a header declares."""
    src = open(os.path.join(ROOT, "include", header)).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return set(re.findall(r"\b(ns_[a-z0-9_]+)\s*\(", src))


def test_library_exports_every_declared_symbol(handle):
    declared = _declared("ns.h") | _declared("ns_attn.h") | _declared("ns_mla.h") | _declared("ns_pre.h")
    assert len(_declared("ns.h")) == 26                      # the reference's 26 (kernels/ns/ns.h:18-56)
    missing = [n for n in sorted(declared) if not hasattr(handle, n)]
    assert not missing, missing
    # and the host tables bind exactly the declared set
    assert set(NS_H) == _declared("ns.h")
    assert set(ATTN_H) == _declared("ns_attn.h")
    assert set(MLA_H) == _declared("ns_mla.h")
    assert set(PRE_H) == _declared("ns_pre.h")


def test_pure_functions_without_a_gpu(handle):
    f = handle.ns_attn_decode_scratch
    f.restype, f.argtypes = C.c_int64, [C.c_int64] * 6
    # one row, 32 / 8 heads, 4096 keys: splits of 128 -> 32 partials of D + 2 floats a head
    assert f(1, 32, 8, 128, 4095, 0) == 32 * 32 * 130
    assert f(0, 32, 8, 128, 4095, 0) == 0
    # heads of 256 aim for half as many work-groups: 32768 keys x 2 heads in 256 splits of 256 keys -> 128 a head; heads of
    # 128 are sized for the cache form that splits finest (q4_0 rows: 512 work-groups, but 256 of them first while a split
    # stays within 512 keys -> 128 a head here, 256 a head of 512 keys at four times the keys)
    assert f(1, 16, 2, 256, 32767, 0) == 16 * 128 * 258 and f(1, 16, 2, 128, 32767, 0) == 16 * 128 * 130
    assert f(1, 16, 2, 128, 131071, 0) == 16 * 256 * 130
    # a verify pass needs at least its rows' own
    assert f(4, 32, 4, 128, 65536, 0) >= 4 * f(1, 32, 4, 128, 65536, 0)
    # a window bounds the splits whatever the position
    assert f(1, 16, 1, 128, 10 ** 6, 2048) <= 16 * 17 * 130
    s = handle.ns_q35_attn_decode_supported
    s.restype, s.argtypes = C.c_int, [C.c_int64] * 4
    assert s(1, 12, 2, 256) == 1 and s(8, 32, 8, 128) == 1 and s(17, 32, 8, 128) == 0 and s(1, 12, 5, 128) == 0 and s(1, 12, 2, 96) == 0
    p = handle.ns_mg_attn_prompt_supported
    p.restype, p.argtypes = C.c_int, [C.c_int64] * 4
    assert p(17, 64, 4, 128) == 1 and p(16, 64, 4, 128) == 0 and p(100, 64, 4, 256) == 1 and p(100, 64, 4, 64) == 0
    m = handle.ns_mla_decode_latent_scratch
    m.restype, m.argtypes = C.c_int64, [C.c_int64] * 3
    assert m(1, 128, 32767) == 128 * 128 * 260 and m(0, 128, 5) == 0     # two 64-row groups x 128 splits of 256 cells; a partial: 512 halfs + m, l (+ 2)
    assert m(2, 128, 32766) == 256 * 128 * 260                           # two 128-row groups x 128 splits
    # whole rounds of an XCD's 32 places: 3 row groups take 79 splits (10 an XCD = 30 work-groups; 86 would be 11 = 33, a
    # second round for three of them), 5 groups 47; 17 rows end at 16 groups x 16 splits, the 17th row a pass of its own; 33
    # groups, fewer than 8 splits, are dealt over the whole chip: 7 splits = 231 work-groups
    assert m(3, 128, 131069) == 3 * 128 * 79 * 260 and m(5, 128, 32763) == 5 * 128 * 47 * 260
    assert m(17, 128, 32751) == m(16, 128, 32751) == 16 * 128 * 16 * 260 and m(33, 128, 32735) == 33 * 128 * 7 * 260
    handle.ns_version.restype = C.c_char_p
    assert b"gfx950" in handle.ns_version()
    handle.ns_last_error.restype = C.c_char_p
    assert handle.ns_last_error() is not None


def test_null_buffers_are_refused_before_any_launch(handle):
    """Entry points that launch kernels check their pointers and strides on the host: a forgotten buffer is -1 with the
    reason, not a GPU fault. (No ns_gpu here either: nothing may touch the device before the checks pass.)"""
    i64, P, f32 = C.c_int64, C.c_void_p, C.c_float
    handle.ns_last_error.restype = C.c_char_p
    buf = C.create_string_buffer(4096)
    b = C.addressof(buf) // 16 * 16 + 16

    def refused(name, argtypes, args, word):
        f = getattr(handle, name)
        f.restype, f.argtypes = C.c_int, argtypes
        assert f(*args) == -1, name
        assert word in handle.ns_last_error().decode(), (name, handle.ns_last_error())

    st = [P, C.c_int, C.c_int, P, i64, P, i64, i64, i64, i64, i64, i64, P, P]
    refused("ns_attn_kv_store", st, (None, 0, 0, b, 128, b, 128, 1, 1, 128, 4, 0, b, None), "null")
    refused("ns_attn_kv_store", st, (None, 0, 0, None, 128, b, 128, 1, 1, 128, 4, 0, b, b), "null")
    refused("ns_attn_kv_dequant", [P, C.c_int, P, i64, i64, i64, P], (None, 1, b, 2, 128, 136, None), "null")
    refused("ns_attn_kv_dequant", [P, C.c_int, P, i64, i64, i64, P], (None, 1, b, 2, 128, 100, b), "a row apart")
    refused("ns_q35_fwht32", [P, P, i64, i64, i64], (None, None, 2, 64, 64), "null")
    refused("ns_q35_fwht32", [P, P, i64, i64, i64], (None, b, 2, 64, 32), "a row apart")
    ds = [P, P, P, f32, P, i64, i64, i64, i64, f32, f32, f32, f32, f32, f32]
    refused("ns_ds2_kv_store", ds, (None, b, None, 1e-6, b, 1, 512, 64, 0, 1e4, 1.0, 0.0, 1.0, 0.0, 0.0), "null")
    refused("ns_to_q8row", [P, P, P, i64, i64], (None, b, None, 1, 512), "null")
    refused("ns_gather_q8_h", [P, P, P, P, i64, i64], (None, b, None, b, 1, 512), "null")
    refused("ns_gather_q8_h", [P, P, P, P, i64, i64], (None, b, b, b, 1, 256), "512")
    refused("ns_mla_cells", [P, P, P, i64, i64, i64, P, P, i64], (None, None, None, 2, 0, 5, b, None, 64), "null")
    refused("ns_mla_cells", [P, P, P, i64, i64, i64, P, P, i64], (None, None, b, 2, 4, 5, b, b, 64), "no lists")
    refused("ns_softmax_masked", [P, P, i64, i64, i64, P, f32], (None, b, 2, 4, 64, None, 1.0), "null")
    gm = [P, i64, i64, i64, P, i64, P, P, i64, C.c_int]
    refused("ns_gemm_f16", gm, (None, 4, 4, 64, b, 64, None, b, 4, 0), "null")
    refused("ns_gemm_f16", gm, (None, 4, 4, 64, b, 32, b, b, 4, 0), "apart")
    gb = [P, i64, C.c_int, i64, i64, i64, P, i64, i64, P, i64, i64, P, i64, i64, C.c_int]
    refused("ns_gemm_batch_h", gb, (None, 2, 0, 4, 8, 64, b, 64, 0, b, 4, 0, b, 8, 0, 0), "apart")
    refused("ns_gemm_batch_h", gb, (None, 2, 1, 4, 8, 64, b, 64, 0, b, 64, 0, None, 8, 0, 0), "null")
    refused("ns_to_f16", [P, P, P, i64], (None, b, None, 5), "null")
    refused("ns_gather_h", [P, P, P, P, i64, i64], (None, b, None, b, 4, 512), "null")
    refused("ns_gather_h", [P, P, P, P, i64, i64], (None, b, b, b, 4, 100), "multiple of 8")
    refused("ns_attn_tune", [C.c_int, i64], (9, 1), "knob")
    refused("ns_attn_tune", [C.c_int, i64], (0, -1), "knob")
    handle.ns_attn_tune.restype = C.c_int
    assert handle.ns_attn_tune(0, 0) == 0
    # the new pure functions
    bs = handle.ns_mg_attn_block_scratch
    bs.restype, bs.argtypes = i64, [i64] * 6
    ds_ = handle.ns_attn_decode_scratch
    ds_.restype, ds_.argtypes = i64, [i64] * 6
    assert bs(8, 32, 8, 128, 5000, 4096) == ds_(8, 32, 8, 128, 5000, 4096) and bs(17, 32, 8, 128, 5000, 0) == 0
    sup = handle.ns_mm3s_attend_supported
    sup.restype, sup.argtypes = C.c_int, [i64] * 3
    assert sup(64, 4, 128) == 1 and sup(64, 4, 64) == 0 and sup(63, 4, 128) == 0


def test_row_bytes_and_errors():
    assert [kv_row_bytes(k, 128) for k in (0, 1, 2, 3)] == [256, 136, 72, 256]
    assert [kv_row_bytes(k, 256) for k in (0, 1, 2)] == [512, 272, 144]      # llm/qwen35/src/engine.rs:54-60
    with pytest.raises(Error):
        kv_row_bytes(4, 128)
    # crates/core/src/lib.rs:509-516
    assert Error("copying to the GPU: hip: hipMemcpyAsync: hipErrorOutOfMemory").is_no_room()
    assert Error("device allocation of 1024 bytes failed").is_no_room()
    assert Error.no_room("needs 2.0 GiB more").is_no_room()
    assert not Error("hip: hipStreamSynchronize: unspecified launch failure").is_no_room()


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    from nextsycl_amd.sys import Api
    monkeypatch.setenv("NEXTSYCL_LIB", str(tmp_path / "nope.so"))
    with pytest.raises(OSError):
        Api()


def test_product_never_imports_the_oracle():
    """The oracle is test infrastructure: nothing under nextsycl_amd/ may import, load or link it."""
    for dirpath, _, files in os.walk(os.path.join(ROOT, "nextsycl_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".hpp", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src and "liboracle" not in src, os.path.join(dirpath, f)


def test_bench_draws_its_inputs_from_the_fixed_generator():
    """bench.py's inputs come from the generator the tests use - xorshift64* -> Box-Muller, stated once in the oracle and
    once, independently, in bench_inputs.c: the same bits. A matrix is a stream every 1024 rows, seeded seed + first row."""
    import numpy as np

    import bench
    from oracle import orc

    for seed, n, sigma in ((1, 7, 1.0), (0xA11CE, 100001, 0.5), (0xC0FFEE + 8192, 4096, 1.0)):
        assert np.array_equal(bench.randn(seed, (n,), sigma), orc.randn(seed, (n,), sigma))
    x = bench.randn(0xB0B, (2500, 96), 0.5)
    for s0 in (0, 1024, 2048):
        rows = min(1024, 2500 - s0)
        assert np.array_equal(x[s0:s0 + rows].ravel(), orc.randn(0xB0B + s0, (rows * 96,), 0.5))


def test_bench_refuses_more_than_one_gpu():
    """One GPU is what this build runs on: `bench.py --gpus N` with N above 1 exits with a message that says so, before it
    touches the library or a device."""
    import subprocess
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "one GPU" in r.stderr and not r.stdout.strip()
