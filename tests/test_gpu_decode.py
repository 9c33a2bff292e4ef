"""Parity of the split-K decode / verify kernel (ns_attn_decode_t and the reference-named entry points over it)
against the oracle, through the C ABI, on seeded inputs."""
import numpy as np
import pytest

from helpers import check_close, gpu_decode, make_kv, make_q
from nextsycl_amd import DevBuf, Error
from nextsycl_amd.attn import BF16, F16, F32
from oracle import orc

pytestmark = pytest.mark.gpu


SMALL = [
    # T, Hq, Hkv, D, p0, win, kt, qt
    (1, 4, 1, 128, 0, 0, 0, F32),          # one key
    (1, 4, 1, 128, 31, 0, 0, F32),         # one tile exactly
    (1, 4, 1, 128, 32, 0, 0, F32),         # one key into the second tile
    (1, 32, 8, 128, 1000, 0, 0, F16),      # G 4
    (1, 40, 8, 128, 777, 0, 0, F32),       # G 5: no reference instantiation, same algorithm
    (4, 32, 4, 128, 2049, 0, 0, F16),      # a verify pass, G 8: two row tiles
    (16, 16, 1, 128, 300, 0, 0, F32),      # 256 rows of a key head: chunks of two row tiles
    (1, 64, 4, 128, 5000, 0, 1, F16),      # q8_0, G 16
    (2, 12, 2, 128, 3000, 0, 2, F32),      # q4_0
    (3, 8, 2, 128, 4000, 0, 3, BF16),      # bfloat16 cache and rows
    (2, 8, 2, 128, 166, 0, 3, F32),        # bfloat16 cache, float32 rows: the rows in two bfloat16 parts
    (5, 16, 2, 128, 3000, 0, 3, F16),      # ... half rows, two row tiles
    (1, 6, 1, 256, 700, 0, 3, F32),        # ... heads of 256
    (1, 12, 2, 256, 1500, 0, 0, F32),      # qwen35's head size, G 6
    (2, 12, 2, 256, 900, 0, 1, F32),       # ... with a q8_0 cache
    (2, 8, 2, 256, 700, 0, 2, F32),        # ... with a q4_0 cache
    (4, 12, 2, 256, 800, 0, 1, F32),       # ... q8_0 and 24 rows a key head: two row tiles, the whole register file
    (5, 12, 2, 256, 5000, 0, 2, F16),      # ... q4_0 and 30 rows
    (8, 12, 2, 256, 2100, 0, 1, F32),      # ... 48 rows: two chunks of two row tiles
    (4, 16, 2, 128, 1200, 0, 1, F16),      # q8_0, 32 rows a key head: two row tiles
    (1, 8, 2, 128, 5000, 1024, 0, F32),    # a window
    (5, 8, 2, 128, 130, 100, 0, F32),      # a window shorter than a split
]


@pytest.mark.parametrize("T,Hq,Hkv,D,p0,win,kt,qt", SMALL)
def test_decode_small(ops, T, Hq, Hkv, D, p0, win, kt, qt):
    cap = p0 + T + 7
    kc, vc = make_kv(kt, Hkv, D, cap, p0 + T)
    qd, qf = make_q(qt, T, Hq, D)
    got, _ = gpu_decode(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    ref = orc.attn_f64(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(got, ref, qt, "decode vs float64 closed form", kt=kt)
    if kt != 3:
        # and the reference's exact kernel (float32, its own summation order) sits as close to the closed form
        ex = orc.attn_exact(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
        mx, rel, _ = orc.compare(got, ex.astype(np.float64))
        assert mx <= 2e-3 and rel <= 1e-3 + (2.0 ** -9 if qt == BF16 else 0)


def _random_cases(n, seed):
    """Seeded shapes over everything the kernel branches on: rows and groups (one or two row tiles, chunks), head size,
    cache form, context from inside one tile to many splits, windows shorter and longer than a split."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        D = int(rng.choice([128, 128, 256]))
        kt = int(rng.choice([0, 0, 1, 2, 3]))
        Hkv = int(rng.integers(1, 4))
        G = int(rng.choice([1, 2, 3, 4, 8, 16]))
        T = int(rng.choice([1, 1, 2, 3, 5, 8, 16]))
        p0 = int(rng.choice([rng.integers(0, 70), rng.integers(70, 700), rng.integers(700, 6000)]))
        win = int(rng.choice([0, 0, rng.integers(1, 64), rng.integers(64, 2000)]))
        qt = BF16 if kt == 3 else int(rng.choice([F32, F16]))
        out.append((T, Hkv * G, Hkv, D, p0, win, kt, qt))
    return out


@pytest.mark.parametrize("T,Hq,Hkv,D,p0,win,kt,qt", _random_cases(48, 20240607))
def test_decode_seeded_shapes(ops, T, Hq, Hkv, D, p0, win, kt, qt):
    cap = p0 + T + 3
    kc, vc = make_kv(kt, Hkv, D, cap, p0 + T, cfg=p0 % 7)
    qd, qf = make_q(qt, T, Hq, D, cfg=T)
    got, _ = gpu_decode(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    ref = orc.attn_f64(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(got, ref, qt, "decode vs float64 closed form", kt=kt)


def test_decode_ring_wrap(ops):
    """A ring cache that has wrapped: slot = position % cap, window inside the ring."""
    T, Hq, Hkv, D, cap, win = 3, 8, 2, 128, 512, 400
    p0 = 1300
    k = orc.randn(11, (p0 + T, Hkv * D))
    v = orc.randn(12, (p0 + T, Hkv * D))
    kc = np.zeros((Hkv, cap, 2 * D), np.uint8)
    vc = np.zeros((Hkv, cap, 2 * D), np.uint8)
    # positions stored in order: later ones overwrite their slot, as the engine's passes do
    for s in range(0, p0 + T, 100):
        e = min(p0 + T, s + 100)
        orc.kv_store(0, k[s:e], v[s:e], Hkv, D, cap, s, kc, vc, ring=True)
    qd, qf = make_q(F32, T, Hq, D)
    got, _ = gpu_decode(ops, F32, 0, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    ref = orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(got, ref, F32, "ring decode")


def test_decode_position_major(ops):
    """MiniMax-M3's layout [position][G][128] with an explicit scale, against its exact kernel's restatement."""
    T, H, G, pos0, scale = 2, 16, 2, 2500, 0.07
    cap = pos0 + T
    kc, vc = make_kv(0, G, 128, cap, cap, pm=True)
    qd, qf = make_q(F32, T, H, 128)
    got, _ = gpu_decode(ops, F32, 0, qd, kc, vc, T, H, G, 128, cap, pos0, pm=True, scale=scale)
    ref = orc.attn_f64(qf, kc, vc, 0, T, H, G, 128, cap, pos0, pm=True, scale=scale)
    check_close(got, ref, F32, "position-major decode")
    ex = orc.mm3_attend(qf, kc.view(np.uint16), vc.view(np.uint16), T, H, G, pos0, scale)
    check_close(ex, ref, F32, "the exact kernel's restatement itself")
    # the reference-named entry point (no scratch argument: the library's own)
    g = ops.gpu
    qb, ob = DevBuf.of(g, qd), DevBuf(g, T * H * 128 * 4)
    ops.minimaxm3_attend(qb, DevBuf.of(g, kc), DevBuf.of(g, vc), ob, T, H, G, pos0, scale)
    assert np.array_equal(ob.read(np.float32).reshape(T, -1), got)


@pytest.mark.parametrize("kt,G,D", [(0, 8, 128), (1, 16, 128), (2, 4, 128), (3, 5, 128), (0, 6, 256), (1, 6, 256), (2, 6, 256)])
def test_verify_rows_equal_their_one_row_pass(ops, kt, G, D):
    """The reference's spec-check invariant (cli/nextsycl/src/main.rs:967-989): a row's result is the same whatever
    rows share its pass - bit for bit - here across passes of 1, 2, 4 and 8 rows at the same positions."""
    Hkv, Tmax = 2, 8
    Hq = Hkv * G
    for p0 in (4090, 65533):         # the second straddles a split-size step: rows 0,1 and rows 2.. get different splits
        cap = p0 + Tmax
        kc, vc = make_kv(kt, Hkv, D, cap, cap, cfg=kt)
        qd, _ = make_q(F32, Tmax, Hq, D, cfg=kt)
        g = ops.gpu
        bufs = (DevBuf.of(g, kc), DevBuf.of(g, vc))
        full, _ = gpu_decode(ops, F32, kt, qd, kc, vc, Tmax, Hq, Hkv, D, cap, p0, bufs=bufs)
        for T in (1, 2, 4):
            for r0 in range(0, Tmax, T):
                part, _ = gpu_decode(ops, F32, kt, qd[r0:r0 + T], kc, vc, T, Hq, Hkv, D, cap, p0 + r0, bufs=bufs)
                assert np.array_equal(part.view(np.uint32), full[r0:r0 + T].view(np.uint32)), (kt, p0, T, r0)


def test_reference_named_entry_points_agree(ops):
    """ns_q35_attn_decode_kv / ns_mg_attn_decode / ns_q35_attn / ns_mg_attn are the typed kernel behind the reference's
    names: float32 rows, same bits."""
    T, Hq, Hkv, D, p0 = 4, 32, 4, 128, 3001
    cap = p0 + T
    g = ops.gpu
    for kt in (0, 1, 2):
        kc, vc = make_kv(kt, Hkv, D, cap, cap)
        qd, _ = make_q(F32, T, Hq, D)
        bufs = (DevBuf.of(g, kc), DevBuf.of(g, vc))
        want, _ = gpu_decode(ops, F32, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, bufs=bufs)
        qb, ob = DevBuf.of(g, qd), DevBuf(g, T * Hq * D * 4)
        sc = DevBuf(g, 4 * ops.k.q35_attn_decode_scratch(T, Hq, Hkv, D, p0))
        ops.q35_attn_decode_kv(kt, qb, Hq * D, bufs[0], bufs[1], T, Hq, Hkv, D, cap, p0, ob, sc)
        assert np.array_equal(ob.read(np.float32).reshape(T, -1), want)
        if kt == 0:
            for call in ("mg_dec", "mg", "q35"):
                ob.fill(0)
                if call == "mg_dec":
                    ops.mg_attn_decode(qb, bufs[0], bufs[1], T, Hq, Hkv, D, cap, p0, 0, ob, sc)
                elif call == "mg":
                    sc2 = DevBuf(g, 4 * ops.k.mg_attn_scratch(T, Hq, Hkv, D, p0, 0, 1))
                    ops.mg_attn(qb, bufs[0], bufs[1], T, Hq, Hkv, D, cap, p0, 0, True, ob, sc2)
                else:
                    sc2 = DevBuf(g, 4 * ops.k.q35_attn_scratch(T, Hq, Hkv, D, p0))
                    ops.q35_attn(qb, Hq * D, bufs[0], bufs[1], T, Hq, Hkv, D, cap, p0, ob, sc2)
                assert np.array_equal(ob.read(np.float32).reshape(T, -1), want), call


def test_negative_control(ops):
    """A deliberately wrong computation must fail the gate (the reference once had a parity column that measured
    nothing: docs/ports/minimax-m31.md:313): a wrong scale, and keys shifted by one position."""
    T, Hq, Hkv, D, p0 = 1, 8, 2, 128, 2000
    cap = p0 + T
    kc, vc = make_kv(0, Hkv, D, cap, cap)
    qd, qf = make_q(F32, T, Hq, D)
    ref = orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, cap, p0)
    wrong, _ = gpu_decode(ops, F32, 0, qd, kc, vc, T, Hq, Hkv, D, cap, p0, scale=1.02 / np.sqrt(D))
    with pytest.raises(AssertionError):
        check_close(wrong, ref, F32, "wrong scale")
    shifted, _ = gpu_decode(ops, F32, 0, qd, np.roll(kc, 1, axis=1), vc, T, Hq, Hkv, D, cap, p0)
    with pytest.raises(AssertionError):
        check_close(shifted, ref, F32, "shifted keys")
    # and the output buffer really is written by the kernel: it was filled with 0xFF before the call
    good, raw = gpu_decode(ops, F32, 0, qd, kc, vc, T, Hq, Hkv, D, cap, p0)
    check_close(good, ref, F32, "control")


def test_argument_errors(ops):
    g = ops.gpu
    b = DevBuf(g, 1 << 20)
    k = ops.k
    raw = g.raw
    assert k.attn_decode_t(raw, 0, 0, 0, b.ptr, 512, b.ptr, b.ptr, 17, 4, 1, 128, 64, 0, 0, 0.0, b.ptr, b.ptr) == -1
    assert "1..16 rows" in k.api.error()
    assert k.attn_decode_t(raw, 0, 0, 0, b.ptr, 512, b.ptr, b.ptr, 1, 4, 1, 96, 64, 0, 0, 0.0, b.ptr, b.ptr) == -1
    assert "heads of 128 or 256" in k.api.error()
    assert k.attn_decode_t(raw, 0, 0, 0, b.ptr, 512, b.ptr, b.ptr, 1, 5, 2, 128, 64, 0, 0, 0.0, b.ptr, b.ptr) == -1
    assert k.attn_decode_t(raw, 0, 0, 0, b.ptr, 512, b.ptr, b.ptr, 1, 4, 1, 128, 64, 64, 0, 0.0, b.ptr, b.ptr) == -1
    assert "capacity" in k.api.error()
    assert k.attn_decode_t(raw, 0, 0, 0, b.ptr, 512, b.ptr, b.ptr, 1, 4, 1, 128, 64, 0, 0, 0.0, b.ptr, None) == -1
    assert "no scratch" in k.api.error()
    assert k.attn_decode_t(raw, 0, 7, 0, b.ptr, 512, b.ptr, b.ptr, 1, 4, 1, 128, 64, 0, 0, 0.0, b.ptr, b.ptr) == -1
    # zero rows: nothing to do, nothing checked
    assert k.attn_decode_t(raw, 0, 0, 0, None, 0, None, None, 0, 4, 1, 128, 64, 0, 0, 0.0, None, None) == 0
    with pytest.raises(Error):
        ops.decode(F32, 0, DevBuf(g, 16), 512, b, b, 1, 4, 1, 128, 64, 0, b, b)


def test_alternating_shapes_repeat_their_bits(ops):
    """Launches of several shapes alternate on one queue (other split counts, head counts, row tiles, sharing the scratch
    sizes' rule): every launch gives the bits of its shape's first launch, and those are the oracle's rows."""
    g = ops.gpu
    shapes = [(1, 32, 8, 128, 3000), (2, 8, 2, 128, 700), (1, 16, 16, 128, 129), (1, 8, 2, 256, 2500), (4, 32, 4, 128, 2049)]
    state = []
    for i, (T, Hq, Hkv, D, p0) in enumerate(shapes):
        cap = p0 + T
        kc, vc = make_kv(0, Hkv, D, cap, cap, cfg=i)
        qd, qf = make_q(F32, T, Hq, D, cfg=i)
        state.append((T, Hq, Hkv, D, p0, cap, qd, kc, vc, (DevBuf.of(g, kc), DevBuf.of(g, vc)), orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, cap, p0)))
    first = {}
    for rep in range(10):
        for i, (T, Hq, Hkv, D, p0, cap, qd, kc, vc, bufs, ref) in enumerate(state):
            got, raw = gpu_decode(ops, F32, 0, qd, kc, vc, T, Hq, Hkv, D, cap, p0, bufs=bufs)
            if rep == 0:
                first[i] = raw.copy()
                check_close(got, ref, F32, "shape %d" % i)
            else:
                assert np.array_equal(raw, first[i]), "launch %d of shape %d" % (rep, i)
