"""Pins the oracle's checkpoint restatements (ring caches read out in position order, the checkpoint file) without the
reference: against a slot-by-slot brute force written another way (one row a step, no runs), against hand-written file
bytes, and by the round trips the format must close. The host module's file format (no GPU needed) is checked against
the same bytes."""
import io

import numpy as np
import pytest

from nextsycl_amd import Error
from nextsycl_amd.checkpoint import MAGIC, Checkpoint, kept
from oracle import orc


def brute_save(cache, heads, cap, row, w, pos):
    """Row by row: position p of head h is the `row` bytes at slot p % cap."""
    c = cache.reshape(heads, cap, row)
    first = 0 if w == 0 else max(0, pos - w + 1)
    return np.stack([np.stack([c[h, p % cap] for p in range(first, pos)]) if pos > first else np.zeros((0, row), np.uint8)
                     for h in range(heads)]).reshape(-1)


CASES = [  # heads, cap, row, window, position
    (2, 16, 8, 0, 11),       # no window, part of the cache
    (2, 16, 8, 0, 16),       # no window, all of it
    (3, 8, 6, 8, 5),         # a ring not yet wrapped
    (3, 8, 6, 8, 8),         # kept = 1: positions 1..7
    (3, 8, 6, 8, 29),        # wrapped: two runs a head
    (1, 7, 2, 5, 23),        # capacity above the window, odd sizes
    (4, 5, 10, 6, 10),       # window - 1 == capacity: every slot, starting at slot 0
    (2, 9, 4, 3, 0),         # nothing fed
]


@pytest.mark.parametrize("heads,cap,row,w,pos", CASES)
def test_ring_save_is_the_rows_in_position_order(heads, cap, row, w, pos):
    rng = np.random.default_rng(pos * 131 + cap)
    cache = rng.integers(0, 256, heads * cap * row, dtype=np.uint8)
    got = orc.ring_save(cache, heads, cap, row, w, pos)
    assert got.size == heads * (pos - orc.ring_kept(w, pos)) * row
    assert np.array_equal(got, brute_save(cache, heads, cap, row, w, pos))
    assert orc.ring_kept(w, pos) == kept(w, pos)


def test_ring_kept_known_values():
    # w = 0 keeps everything; w > 0 keeps the last w - 1 positions
    assert [orc.ring_kept(0, p) for p in (0, 5, 1000)] == [0, 0, 0]
    assert [orc.ring_kept(4, p) for p in (0, 2, 3, 4, 10)] == [0, 0, 0, 1, 7]
    assert orc.ring_kept(1, 9) == 9


@pytest.mark.parametrize("heads,cap,row,w,pos", CASES)
def test_ring_restore_closes_the_round_trip(heads, cap, row, w, pos):
    rng = np.random.default_rng(7 + pos)
    cache = rng.integers(0, 256, heads * cap * row, dtype=np.uint8)
    b = orc.ring_save(cache, heads, cap, row, w, pos)
    # into a ring of ANOTHER capacity: saved again it gives the same buffer, and slots outside the kept span stay as they were
    cap2 = cap + 3
    other = np.full(heads * cap2 * row, 0xAA, np.uint8)
    orc.ring_restore(other, b, heads, cap2, row, w, pos)
    assert np.array_equal(orc.ring_save(other, heads, cap2, row, w, pos), b)
    first = orc.ring_kept(w, pos)
    touched = {p % cap2 for p in range(first, pos)}
    o = other.reshape(heads, cap2, row)
    for s in range(cap2):
        if s not in touched:
            assert (o[:, s] == 0xAA).all()
    with pytest.raises(ValueError):
        orc.ring_restore(other, b[:-1] if b.size else np.zeros(1, np.uint8), heads, cap2, row, w, pos)


def test_ring_copy_between_capacities():
    heads, row, scap, dcap, first, to = 3, 4, 8, 11, 13, 20
    rng = np.random.default_rng(3)
    src = rng.integers(0, 256, heads * scap * row, dtype=np.uint8)
    dst = np.full(heads * dcap * row, 0x55, np.uint8)
    orc.ring_copy(dst, dcap, src, scap, heads, row, first, to)
    s, d = src.reshape(heads, scap, row), dst.reshape(heads, dcap, row)
    for h in range(heads):
        for p in range(first, to):
            assert np.array_equal(d[h, p % dcap], s[h, p % scap])
    untouched = set(range(dcap)) - {p % dcap for p in range(first, to)}
    assert all((d[:, x] == 0x55).all() for x in untouched)


def test_checkpoint_file_known_bytes():
    # written out by hand: magic, position 3, two buffers (2 bytes, 0 bytes)
    want = (b"NSMG1" + bytes([3, 0, 0, 0, 0, 0, 0, 0]) + bytes([2, 0, 0, 0, 0, 0, 0, 0]) + bytes([2, 0, 0, 0, 0, 0, 0, 0]) + b"\x07\xff"
            + bytes(8))
    bufs = [np.array([7, 255], np.uint8), np.zeros(0, np.uint8)]
    assert orc.checkpoint_file(b"NSMG1", 3, bufs) == want
    assert Checkpoint(3, bufs).to_bytes(MAGIC["museglimmer"]) == want
    # a position past 2^32 keeps all 8 bytes, little-endian
    big = orc.checkpoint_file(b"NSQ35", (1 << 33) + 5, [])
    assert big == b"NSQ35" + bytes([5, 0, 0, 0, 2, 0, 0, 0]) + bytes(8)
    assert Checkpoint((1 << 33) + 5, []).to_bytes(MAGIC["qwen35"]) == big


@pytest.mark.parametrize("arch", sorted(MAGIC))
def test_checkpoint_file_round_trip(arch):
    rng = np.random.default_rng(11)
    bufs = [rng.integers(0, 256, n, dtype=np.uint8) for n in (0, 1, 4096, 777)]
    mtp = (3, 9, [1, 2, 0xFFFFFFFF]) if arch == "glm5next" else None
    ck = Checkpoint(12345, bufs, mtp)
    raw = ck.to_bytes(MAGIC[arch])
    if arch != "glm5next":
        assert raw == orc.checkpoint_file(MAGIC[arch], 12345, bufs)
    else:       # GLM's file: the common form, then the draft block's state
        head = orc.checkpoint_file(MAGIC[arch], 12345, bufs)
        assert raw[:len(head)] == head
        assert raw[len(head):] == (1).to_bytes(8, "little") + (3).to_bytes(8, "little") + (9).to_bytes(8, "little") + (3).to_bytes(8, "little") + \
            bytes([1, 0, 0, 0, 2, 0, 0, 0, 255, 255, 255, 255])
        assert Checkpoint(1, []).to_bytes(MAGIC[arch])[-8:] == bytes(8)
    back = Checkpoint.read_from(io.BytesIO(raw), MAGIC[arch])
    assert back.pos == 12345 and back.bytes == ck.bytes == sum(b.size for b in bufs) and back.mtp == mtp
    assert all(np.array_equal(a, b) for a, b in zip(back.bufs, bufs))
    other = MAGIC["qwen35" if arch != "qwen35" else "ricursive"]
    with pytest.raises(Error, match="not a"):
        Checkpoint.read_from(io.BytesIO(raw), other)
    with pytest.raises(Error, match="ends early"):
        Checkpoint.read_from(io.BytesIO(raw[:-1]), MAGIC[arch])
