"""Checkpoints through the C ABI: the rows-copy kernel, and save / restore / copy_session above it, byte for byte
against the oracle's restatement of the engines' host loops; at full size through what the format must close (a
checkpoint restored into caches of another capacity reads back the same, and attention over them gives the same bits)."""
import io

import numpy as np
import pytest

from helpers import gpu_decode, make_q
from nextsycl_amd import DevBuf, Error
from nextsycl_amd.attn import F16, kv_row_bytes
from nextsycl_amd.checkpoint import MAGIC, Checkpoint, Ring, copy_session, kept, restore, save
from oracle import orc

pytestmark = pytest.mark.gpu


def _bytes(seed, n):
    return np.random.default_rng(seed).integers(0, 256, n, dtype=np.uint8)


# heads, row bytes, source (cap, base), destination (cap, base), positions [from, to)
ROWS = [
    (4, 256, (64, 0), (40, 24), 24, 64),        # half rows of D = 128 (16-byte units): a linear cache into position order
    (4, 256, (48, 0), (30, 70), 70, 100),       # a ring that wraps inside the span
    (2, 136, (50, 0), (64, 0), 37, 87),         # q8_0 rows (8-byte units), ring into a larger ring, both wrap
    (3, 72, (33, 0), (33, 66), 66, 99),         # q4_0 rows, every slot of the ring
    (1, 1152, (200, 0), (77, 123), 123, 200),   # a latent cache's rows (576 halfs), one head
    (1, 544, (90, 0), (90, 0), 10, 55),         # q8 latent rows, same geometry: a plain copy of the span
    (5, 12, (19, 0), (23, 0), 40, 59),          # 4-byte units
    (5, 6, (19, 0), (7, 50), 50, 57),           # 2-byte units
    (2, 256, (16, 0), (1, 31), 31, 32),         # one position
]


@pytest.mark.parametrize("heads,row,src,dst,a,b", ROWS)
def test_rows_copy_matches_oracle(ops, heads, row, src, dst, a, b):
    g = ops.gpu
    (scap, sbase), (dcap, dbase) = src, dst
    s = _bytes(a * 7 + row, heads * scap * row)
    d0 = np.full(heads * dcap * row, 0xC3, np.uint8)
    # the oracle's ring copy places position p at p % cap; a cache with a base is that ring rotated by the base
    want = d0.copy().reshape(heads, dcap, row)
    sv = s.reshape(heads, scap, row)
    for p in range(a, b):
        want[:, (p - dbase) % dcap] = sv[:, (p - sbase) % scap]
    if sbase == 0 and dbase == 0:       # both rings: the engines' copy_ring itself
        viaring = d0.copy()
        orc.ring_copy(viaring, dcap, s, scap, heads, row, a, b)
        assert np.array_equal(viaring.reshape(want.shape), want)
    if sbase == 0 and dbase == a and dcap == b - a:   # ring into position order: the engines' save
        assert np.array_equal(orc.ring_save(s, heads, scap, row, 0, b).reshape(heads, b, row)[:, a:].reshape(-1), want.reshape(-1))
    sb, db = DevBuf.of(g, s), DevBuf.of(g, d0)
    ops.kv_rows_copy(sb, scap, sbase, db, dcap, dbase, heads, row, a, b)
    assert np.array_equal(db.read(np.uint8).reshape(want.shape), want)
    assert np.array_equal(sb.read(np.uint8), s)


def test_rows_copy_unaligned_views_fall_to_narrower_units(ops):
    """Caches at an address that is only 2 bytes aligned: the same bytes through 2-byte units."""
    g = ops.gpu
    heads, row, cap, a, b = 2, 256, 20, 3, 17
    s = _bytes(5, 2 + heads * cap * row)
    sb, db = DevBuf.of(g, s), DevBuf(g, 6 + heads * (b - a) * row)
    db.fill(0)
    ops.kv_rows_copy(sb.view(2, heads * cap * row), cap, 0, db.view(6, heads * (b - a) * row), b - a, a, heads, row, a, b)
    want = s[2:].reshape(heads, cap, row)[:, a:b].reshape(-1)
    got = db.read(np.uint8)
    assert np.array_equal(got[6:], want) and not got[:6].any()


def test_rows_copy_rejects(ops):
    g = ops.gpu
    buf = DevBuf(g, 4096)
    with pytest.raises(Error, match="more positions than a cache has slots"):
        ops.kv_rows_copy(buf, 8, 0, buf, 4, 0, 1, 16, 0, 5)
    with pytest.raises(Error, match="even number of bytes"):
        ops.kv_rows_copy(buf, 8, 0, buf, 8, 0, 1, 15, 0, 5)
    with pytest.raises(Error, match="at or past each cache's first"):
        ops.kv_rows_copy(buf, 8, 0, buf, 8, 4, 1, 16, 2, 5)
    with pytest.raises(Error, match="needs"):       # the wrapper's own size check: the source is too small
        ops.kv_rows_copy(buf, 1 << 20, 0, buf, 8, 0, 1, 16, 0, 5)
    ops.kv_rows_copy(buf, 8, 0, buf, 8, 0, 1, 16, 5, 5)       # an empty span is no work


def _session(g, layers, seed, fill=None):
    """[(Ring, host copies of its caches)] for layers of (heads, cap, window, row bytes)."""
    out = []
    for i, (heads, cap, w, row) in enumerate(layers):
        host = [_bytes(seed + 10 * i + j, heads * cap * row) if fill is None else np.full(heads * cap * row, fill, np.uint8) for j in range(2)]
        out.append((Ring(tuple(DevBuf.of(g, h) for h in host), cap, heads, w, row), host))
    return out


LAYERS = [(4, 96, 0, 256), (4, 40, 33, 256), (2, 96, 0, 136), (8, 64, 64, 72), (1, 96, 0, 1152)]


@pytest.mark.parametrize("pos", [0, 1, 31, 32, 77, 96])
def test_save_is_the_oracles_buffers_and_file(ops, pos):
    g = ops.gpu
    sess = _session(g, LAYERS, 100 + pos)
    ck = save(ops, [r for r, _ in sess], pos)
    want = [orc.ring_save(h, r.heads, r.cap, r.row, r.win, pos) for r, host in sess for h in host]
    assert ck.pos == pos and len(ck.bufs) == len(want) == 2 * len(LAYERS)
    for got, w in zip(ck.bufs, want):
        assert np.array_equal(got, w)
    assert ck.bytes == sum(w.size for w in want)
    assert ck.to_bytes(MAGIC["museglimmer"]) == orc.checkpoint_file(b"NSMG1", pos, want)
    # the caches themselves are as they were
    for r, host in sess:
        for c, h in zip(r.bufs, host):
            assert np.array_equal(c.read(np.uint8), h)


@pytest.mark.parametrize("pos", [1, 40, 77])
def test_restore_into_other_capacities(ops, pos):
    g = ops.gpu
    sess = _session(g, LAYERS, 300 + pos)
    ck = Checkpoint.read_from(io.BytesIO(save(ops, [r for r, _ in sess], pos).to_bytes()))     # through the file form
    bigger = [(h, cap + 29, w, row) for h, cap, w, row in LAYERS]
    dst = _session(g, bigger, 0, fill=0x11)
    assert restore(ops, [r for r, _ in dst], 200, ck) == pos
    for (r, host), b_k, b_v in zip(dst, ck.bufs[0::2], ck.bufs[1::2]):
        for c, h, b in zip(r.bufs, host, (b_k, b_v)):
            want = h.copy()
            orc.ring_restore(want, b, r.heads, r.cap, r.row, r.win, pos)
            assert np.array_equal(c.read(np.uint8), want)
    # saved again from the other geometry: the same checkpoint
    again = save(ops, [r for r, _ in dst], pos)
    assert again.to_bytes() == ck.to_bytes()


def test_restore_errors(ops):
    g = ops.gpu
    sess = _session(g, LAYERS, 500)
    rings = [r for r, _ in sess]
    ck = save(ops, rings, 50)
    with pytest.raises(Error, match="a checkpoint of 50 tokens into a session of 49"):
        restore(ops, rings, 49, ck)
    with pytest.raises(Error, match="a short checkpoint"):
        restore(ops, rings, 96, Checkpoint(50, ck.bufs[:-1]))
    with pytest.raises(Error, match="a checkpoint of another shape"):
        restore(ops, rings, 96, Checkpoint(50, ck.bufs[:3] + [ck.bufs[3][:-2]] + ck.bufs[4:]))
    with pytest.raises(Error, match="positions kept in a cache"):
        save(ops, [Ring(rings[0].bufs, 96, 4, 0, 256)], 97)


def test_copy_session_matches_oracle(ops):
    g = ops.gpu
    pos = 83
    src = _session(g, LAYERS, 700)
    other = [(h, cap + 7, w, row) for h, cap, w, row in LAYERS]
    dst = _session(g, other, 0, fill=0x77)
    assert copy_session(ops, [r for r, _ in dst], 200, [r for r, _ in src], pos) == pos
    for (d, dh), (s, sh) in zip(dst, src):
        for c, h0, hs in zip(d.bufs, dh, sh):
            want = h0.copy()
            orc.ring_copy(want, d.cap, hs, s.cap, d.heads, d.row, kept(d.win, pos), pos)
            assert np.array_equal(c.read(np.uint8), want)
    with pytest.raises(Error, match="a session of 83 tokens into one of 82"):
        copy_session(ops, [r for r, _ in dst], 82, [r for r, _ in src], pos)


def test_attention_over_restored_ring_is_bit_identical(ops):
    """A sliding-window session checkpointed, restored into caches of another capacity, decoded: the same output bits
    (the kernel's grouping of keys depends on positions, not slots)."""
    g = ops.gpu
    Hq, Hkv, D, win, cap, cap2, pos = 8, 2, 128, 256, 300, 417, 1000
    T = 2
    k = orc.randn(1, (pos + T, Hkv * D)); v = orc.randn(2, (pos + T, Hkv * D))
    rb = kv_row_bytes(0, D)
    kc, vc = DevBuf(g, Hkv * cap * rb), DevBuf(g, Hkv * cap * rb)
    kc.fill(0); vc.fill(0)
    def feed(kcb, vcb, c, a, b):
        for p0 in range(a, b, 100):         # passes no longer than the ring
            n = min(100, b - p0)
            ops.kv_store(0, DevBuf.of(g, k[p0:p0 + n]), Hkv * D, DevBuf.of(g, v[p0:p0 + n]), Hkv * D, n, Hkv, D, c, p0, kcb, vcb, ring=True)

    feed(kc, vc, cap, 0, pos)
    ck = save(ops, [Ring((kc, vc), cap, Hkv, win, rb)], pos)
    assert ck.bytes == 2 * Hkv * (win - 1) * rb
    kc2, vc2 = DevBuf(g, Hkv * cap2 * rb), DevBuf(g, Hkv * cap2 * rb)
    kc2.fill(0xFF); vc2.fill(0xFF)          # NaN patterns wherever the checkpoint does not write
    assert restore(ops, [Ring((kc2, vc2), cap2, Hkv, win, rb)], 4096, ck) == pos
    feed(kc, vc, cap, pos, pos + T)         # the pass after the checkpoint, into both sessions
    feed(kc2, vc2, cap2, pos, pos + T)
    qd, _ = make_q(F16, T, Hq, D)
    _, a = gpu_decode(ops, F16, 0, qd, None, None, T, Hq, Hkv, D, cap, pos, win=win, bufs=(kc, vc))
    _, b = gpu_decode(ops, F16, 0, qd, None, None, T, Hq, Hkv, D, cap2, pos, win=win, bufs=(kc2, vc2))
    assert np.array_equal(a, b)
    assert np.isfinite(orc.h2f(a)).all()


def test_full_size_round_trip(ops):
    """131072 positions of q8_0 rows, 8 heads (the long-context decode configuration's cache): saved, restored into a
    zeroed cache of another capacity, read back."""
    g = ops.gpu
    heads, cap, row, pos = 8, 131072, 136, 131072
    host = _bytes(9, heads * cap * row)
    c = DevBuf.of(g, host)
    ck = save(ops, [Ring((c,), cap, heads, 0, row)], pos)
    assert ck.bytes == host.size and np.array_equal(ck.bufs[0], host)
    cap2 = cap + 1000
    d = DevBuf(g, heads * cap2 * row)
    d.fill(0)
    assert restore(ops, [Ring((d,), cap2, heads, 0, row)], cap2, ck) == pos
    back = d.read(np.uint8).reshape(heads, cap2, row)
    assert np.array_equal(back[:, :cap].reshape(-1), host) and not back[:, cap:].any()
