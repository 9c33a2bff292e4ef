"""Byte-exact parity of the KV-cache stores, the dequantizing read and the Hadamard rotation against the oracle."""
import numpy as np
import pytest

from nextsycl_amd import DevBuf
from nextsycl_amd.attn import kv_row_bytes
from oracle import orc

pytestmark = pytest.mark.gpu


def _edge_rows(T, n, seed):
    """Rows with the cases a quantizer can get wrong: ties at .5 of a step, zeros, a block of one value, tiny and
    large magnitudes, equal extremes of both signs."""
    x = orc.randn(seed, (T, n))
    x[0, :32] = 0.0                                    # an all-zero block: d = 0, every q = 0
    x[0, 32:64] = np.arange(-16, 16, dtype=np.float32) / 2.0 * (127.0 / 127.0)   # halves: x.5 ties when d = 1/..
    x[0, 32] = 127.0                                   # amax 127 -> d = 1 -> q = round(x), ties away from zero
    x[1, :32] = -3.25
    x[1, 32:64] = 1e-30
    x[1, 64:96] = 6e4
    x[2, :32] = np.where(np.arange(32) % 2 == 0, 2.0, -2.0)   # equal magnitudes, both signs: q4_0 keeps the first
    x[2, 32:64] = np.where(np.arange(32) % 2 == 0, -2.0, 2.0)
    return x


@pytest.mark.parametrize("kt", [0, 3, 1, 2])
@pytest.mark.parametrize("D,Hkv", [(128, 4), (256, 2)])
def test_store_matches_oracle_bytes(ops, kt, D, Hkv):
    g = ops.gpu
    T, cap, p0 = 37, 64, 11
    k = _edge_rows(T, Hkv * D, 21)
    v = _edge_rows(T, Hkv * D, 22)[::-1].copy()
    rb = kv_row_bytes(kt, D)
    kc0 = np.full((Hkv, cap, rb), 0xA5, np.uint8)
    vc0 = np.full((Hkv, cap, rb), 0x5A, np.uint8)
    want_k, want_v = orc.kv_store(kt, k, v, Hkv, D, cap, p0, kc0.copy(), vc0.copy())
    kb, vb = DevBuf.of(g, kc0), DevBuf.of(g, vc0)
    ops.kv_store(kt, DevBuf.of(g, k), Hkv * D, DevBuf.of(g, v), Hkv * D, T, Hkv, D, cap, p0, kb, vb)
    assert np.array_equal(kb.read(np.uint8).reshape(want_k.shape), want_k)
    assert np.array_equal(vb.read(np.uint8).reshape(want_v.shape), want_v)
    # the reference-named entry points write the same bytes
    kb2, vb2 = DevBuf.of(g, kc0), DevBuf.of(g, vc0)
    if kt == 0:
        ops.q35_kv_store(DevBuf.of(g, k), Hkv * D, DevBuf.of(g, v), Hkv * D, T, Hkv, D, cap, p0, kb2, vb2)
    elif kt in (1, 2):
        ops.q35_kv_store_q(kt, DevBuf.of(g, k), Hkv * D, DevBuf.of(g, v), Hkv * D, T, Hkv, D, cap, p0, kb2, vb2)
    if kt != 3:
        assert np.array_equal(kb2.read(np.uint8).reshape(want_k.shape), want_k)
        assert np.array_equal(vb2.read(np.uint8).reshape(want_v.shape), want_v)


def test_store_row_strides(ops):
    """k and v rows further apart than their width (the engines pass views of a wider projection)."""
    g = ops.gpu
    T, Hkv, D, cap, ks, vs = 5, 2, 128, 16, 400, 512
    kw, vw = orc.randn(1, (T, ks)), orc.randn(2, (T, vs))
    for kt in (0, 1, 2):
        rb = kv_row_bytes(kt, D)
        kb, vb = DevBuf(g, Hkv * cap * rb), DevBuf(g, Hkv * cap * rb)
        kb.fill(0)
        vb.fill(0)
        ops.kv_store(kt, DevBuf.of(g, kw), ks, DevBuf.of(g, vw), vs, T, Hkv, D, cap, 3, kb, vb)
        want_k, want_v = orc.kv_store(kt, kw[:, :Hkv * D], vw[:, :Hkv * D], Hkv, D, cap, 3)
        assert np.array_equal(kb.read(np.uint8).reshape(want_k.shape), want_k)
        assert np.array_equal(vb.read(np.uint8).reshape(want_v.shape), want_v)


def test_ring_store(ops):
    g = ops.gpu
    T, Hkv, D, cap, p0 = 9, 2, 128, 12, 20     # slots 8..11, 0..4: wraps
    k, v = orc.randn(5, (T, Hkv * D)), orc.randn(6, (T, Hkv * D))
    kb, vb = DevBuf(g, Hkv * cap * 2 * D), DevBuf(g, Hkv * cap * 2 * D)
    kb.fill(0)
    vb.fill(0)
    ops.mg_kv_store(DevBuf.of(g, k), DevBuf.of(g, v), T, Hkv, D, cap, p0, kb, vb)
    want_k, want_v = orc.kv_store(0, k, v, Hkv, D, cap, p0, ring=True)
    assert np.array_equal(kb.read(np.uint8).reshape(want_k.shape), want_k)
    assert np.array_equal(vb.read(np.uint8).reshape(want_v.shape), want_v)


@pytest.mark.parametrize("kt", [0, 1, 2, 3])
def test_dequant_every_scale(ops, kt):
    """The widening read against the oracle, bit for bit; quantized rows carry every half bit pattern as a scale in
    turn (Inf / NaN scales excluded: a store never writes them)."""
    g = ops.gpu
    D = 128
    rb = kv_row_bytes(kt, D)
    rng = np.random.default_rng(3)
    if kt in (0, 3):
        n = 65536 // D
        rows = np.arange(65536, dtype=np.uint16).view(np.uint8).reshape(n, rb).copy()
    else:
        scales = np.array([b for b in range(65536) if (b & 0x7c00) != 0x7c00], np.uint16)
        n = (scales.size + 3) // 4
        rows = rng.integers(0, 256, (n, rb), dtype=np.uint8)
        sc = np.resize(scales, n * 4).reshape(n, 4)
        rows[:, rb - 8:] = sc.view(np.uint8).reshape(n, 8)
    out = DevBuf(g, n * D * 4)
    ops.kv_dequant(kt, DevBuf.of(g, rows), n, D, out)
    got = out.read(np.float32).reshape(n, D)
    want = orc.kv_dequant(rows, kt, D)
    same = (got.view(np.uint32) == want.view(np.uint32)) | (np.isnan(got) & np.isnan(want))
    assert same.all()


def test_store_capacity_errors(ops):
    g = ops.gpu
    b = DevBuf(g, 1 << 16)
    k = ops.k
    assert k.q35_kv_store(g.raw, b.ptr, 128, b.ptr, 128, 2, 1, 128, 4, 3, b.ptr, b.ptr) == -1
    assert "capacity" in k.api.error()
    assert k.q35_kv_store_q(g.raw, 3, b.ptr, 128, b.ptr, 128, 1, 1, 128, 4, 0, b.ptr, b.ptr) == -1
    assert k.mg_kv_store(g.raw, b.ptr, b.ptr, 5, 1, 128, 4, 0, b.ptr, b.ptr) == -1
    assert k.q35_kv_store(g.raw, None, 0, None, 0, 0, 1, 128, 4, 0, None, None) == 0


def test_fwht32(ops):
    g = ops.gpu
    rows, n, stride = 7, 96, 128
    x = orc.randn(9, (rows, stride))
    xb = DevBuf.of(g, x)
    ops.fwht32(xb, rows, n, stride)
    got = xb.read(np.float32).reshape(rows, stride)
    want = x.copy()
    want[:, :n] = orc.fwht32(np.ascontiguousarray(x[:, :n]))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # its own inverse (to rounding)
    ops.fwht32(xb, rows, n, stride)
    assert np.abs(xb.read(np.float32).reshape(rows, stride) - x).max() < 1e-5
