"""Parity of the causal flash-attention prefill kernel (ns_attn_prompt_t and the reference-named entry points over it)
against the oracle's float64 closed form, through the C ABI, on seeded inputs."""
import numpy as np
import pytest

from helpers import check_close, gpu_decode, gpu_prompt, make_kv, make_q
from nextsycl_amd import DevBuf
from nextsycl_amd.attn import BF16, F16, F32, TUNE_PREFILL_SPLITS, TUNE_PREFILL_WAVES
from oracle import orc

pytestmark = pytest.mark.gpu

SMALL = [
    # T, Hq, Hkv, p0, win, kt, qt
    (17, 4, 1, 0, 0, 0, F32),        # the shortest prompt pass
    (128, 4, 2, 0, 0, 0, F32),       # one row block exactly
    (129, 4, 2, 0, 0, 0, F16),       # one row into the second
    (300, 10, 2, 0, 0, 3, BF16),     # G 5, bfloat16 cache and rows (BASELINE config 2's types)
    (200, 8, 2, 1000, 0, 0, F32),    # a later chunk of a prompt: p0 > 0
    (333, 16, 1, 77, 0, 0, F16),     # G 16 (museglimmer's ratio)
    (260, 4, 1, 500, 256, 0, F32),   # a window
    (96, 6, 6, 31, 0, 3, F32),       # G 1
]


@pytest.mark.parametrize("T,Hq,Hkv,p0,win,kt,qt", SMALL)
def test_prefill_small(ops, T, Hq, Hkv, p0, win, kt, qt):
    D = 128
    cap = p0 + T + 5
    kc, vc = make_kv(kt, Hkv, D, cap, p0 + T)
    qd, qf = make_q(qt, T, Hq, D)
    got, _ = gpu_prompt(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    ref = orc.attn_f64(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(got, ref, qt, "prefill vs float64 closed form", kt=kt)


def _random_cases(n, seed):
    """Seeded shapes over what the kernel branches on: rows around the block sizes, groups, head size, every cache form
    (q8_0 / q4_0 rows of 128 values are 136 / 72 bytes: 8-byte aligned chunks), a context before the pass, windows shorter
    and longer than a tile and than the pass."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        D = int(rng.choice([128, 128, 256]))
        kt = int(rng.choice([0, 3, 1, 2]))
        Hkv = int(rng.integers(1, 3))
        G = int(rng.choice([1, 2, 4, 5, 8]))
        T = int(rng.choice([rng.integers(17, 70), rng.integers(70, 300), rng.integers(300, 600)]))
        p0 = int(rng.choice([0, rng.integers(1, 100), rng.integers(100, 900)]))
        win = int(rng.choice([0, 0, rng.integers(1, 64), rng.integers(64, 700)]))
        qt = BF16 if kt == 3 else int(rng.choice([F32, F16]))
        out.append((T, Hkv * G, Hkv, D, p0, win, kt, qt))
    return out


@pytest.mark.parametrize("T,Hq,Hkv,D,p0,win,kt,qt", _random_cases(32, 20240608))
def test_prefill_seeded_shapes(ops, T, Hq, Hkv, D, p0, win, kt, qt):
    cap = p0 + T + 5
    kc, vc = make_kv(kt, Hkv, D, cap, p0 + T, cfg=T % 5)
    qd, qf = make_q(qt, T, Hq, D, cfg=p0 % 3)
    got, _ = gpu_prompt(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    ref = orc.attn_f64(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(got, ref, qt, "prefill vs float64 closed form", kt=kt)


@pytest.mark.parametrize("T,Hq,Hkv,D,p0,win,kt,qt", [(700, 10, 2, 128, 300, 0, 3, BF16), (513, 4, 1, 128, 0, 400, 0, F32),
                                                     (300, 8, 2, 256, 100, 0, 3, BF16), (260, 4, 1, 256, 0, 200, 0, F32),
                                                     (200, 4, 2, 256, 60, 0, 1, F16), (140, 4, 1, 256, 0, 0, 2, F32)])
def test_prefill_work_groups_of_8_waves(ops, tune, T, Hq, Hkv, D, p0, win, kt, qt):
    """Long passes run work-groups of 8 waves (blocks of 256 rows; 128 at head size 256), short ones of 4: the same rows,
    keys and order of a wave's arithmetic, so the two agree bit for bit; forced here on shapes the oracle finishes in
    seconds."""
    cap = p0 + T + 5
    kc, vc = make_kv(kt, Hkv, D, cap, p0 + T)
    qd, qf = make_q(qt, T, Hq, D)
    tune(TUNE_PREFILL_WAVES, 8)
    got8, _ = gpu_prompt(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    tune(TUNE_PREFILL_WAVES, 4)
    got4, _ = gpu_prompt(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    ref = orc.attn_f64(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(got8, ref, qt, "prefill (8 waves) vs float64 closed form", kt=kt)
    assert np.array_equal(got8, got4)


QROWS128 = [
    # T, Hq, Hkv, p0, win, kt, qt        q8_0 / q4_0 rows of 128 values: both work-group sizes, a window, key splits
    (17, 4, 1, 0, 0, 1, F32),
    (700, 16, 2, 300, 0, 1, F16),        # blocks of 256 rows (8 waves)
    (700, 16, 2, 300, 0, 2, F16),        # q4_0: 4 waves always
    (260, 8, 2, 1000, 200, 1, F32),
    (150, 4, 1, 64, 0, 2, F32),
    (64, 8, 1, 9000, 0, 1, F16),         # key splits
    (64, 8, 1, 9000, 0, 2, F32),
]


@pytest.mark.parametrize("T,Hq,Hkv,p0,win,kt,qt", QROWS128)
def test_prefill_quantized_rows_of_128(ops, T, Hq, Hkv, p0, win, kt, qt):
    D = 128
    cap = p0 + T + 1                     # (an odd row count: the second cache starts 8 bytes off a 16-byte boundary)
    kc, vc = make_kv(kt, Hkv, D, cap, p0 + T)
    qd, qf = make_q(qt, T, Hq, D)
    got, _ = gpu_prompt(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    ref = orc.attn_f64(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(got, ref, qt, "prefill, q8_0 / q4_0 rows of 128", kt=kt)


SPLIT = [
    # T, Hq, Hkv, D, p0, win, kt, qt: few row blocks over many keys - the pass is cut into key splits and merged
    (64, 8, 2, 128, 5000, 0, 0, F16),
    (33, 4, 4, 128, 12000, 0, 3, BF16),
    (300, 4, 1, 128, 9000, 3000, 0, F32),       # a window: the splits start at its first key
    (40, 4, 2, 256, 4000, 0, 0, F32),
    (130, 6, 2, 256, 2500, 0, 1, F16),          # quantized rows at head size 256
    (17, 2, 1, 128, 40000, 0, 0, F32),
    # a key head's rows all in one work-group behind 32768 keys and more: the tiles' transfers stream
    (20, 4, 1, 128, 33000, 0, 3, BF16),         # ... bfloat16 rows kept as they are
    (24, 4, 1, 128, 33000, 0, 3, F32),          # ... float32 query rows over them, in two parts
    (17, 5, 1, 128, 33000, 0, 0, F16),          # ... five heads to an 8-wave work-group
]


@pytest.mark.parametrize("T,Hq,Hkv,D,p0,win,kt,qt", SPLIT)
def test_prefill_key_splits(ops, T, Hq, Hkv, D, p0, win, kt, qt):
    cap = p0 + T + 9
    kc, vc = make_kv(kt, Hkv, D, cap, p0 + T, cfg=3)
    qd, qf = make_q(qt, T, Hq, D, cfg=5)
    got, _ = gpu_prompt(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    ref = orc.attn_f64(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(got, ref, qt, "prefill with key splits vs float64 closed form", kt=kt)


@pytest.mark.parametrize("ns", [2, 5, 16])
@pytest.mark.parametrize("T,Hq,Hkv,D,p0,win", [(200, 4, 2, 128, 0, 0), (150, 2, 1, 128, 700, 90), (70, 4, 2, 256, 333, 0)])
def test_prefill_forced_splits(ops, tune, ns, T, Hq, Hkv, D, p0, win):
    """Splits forced onto short passes: splits wholly past a row block's last key, splits a window leaves empty, a last
    split of a few keys - the same result as the unsplit pass within the path's bar, and the same whatever the
    work-group size (bit for bit)."""
    cap = p0 + T + 1
    kc, vc = make_kv(0, Hkv, D, cap, p0 + T, cfg=1)
    qd, qf = make_q(F32, T, Hq, D, cfg=2)
    ref = orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, cap, p0, win=win)
    tune(TUNE_PREFILL_SPLITS, ns)
    tune(TUNE_PREFILL_WAVES, 8)
    got8, _ = gpu_prompt(ops, F32, 0, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    tune(TUNE_PREFILL_WAVES, 4)
    got4, _ = gpu_prompt(ops, F32, 0, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(got8, ref, F32, "prefill with %d forced splits" % ns)
    assert np.array_equal(got8, got4)


def test_prefill_ring(ops):
    T, Hq, Hkv, D, cap, win, p0 = 150, 4, 2, 128, 512, 300, 900
    k = orc.randn(11, (p0 + T, Hkv * D))
    v = orc.randn(12, (p0 + T, Hkv * D))
    kc = np.zeros((Hkv, cap, 2 * D), np.uint8)
    vc = np.zeros((Hkv, cap, 2 * D), np.uint8)
    for s in range(0, p0 + T, 128):
        e = min(p0 + T, s + 128)
        orc.kv_store(0, k[s:e], v[s:e], Hkv, D, cap, s, kc, vc, ring=True)
    qd, qf = make_q(F32, T, Hq, D)
    got, _ = gpu_prompt(ops, F32, 0, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    ref = orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(got, ref, F32, "ring prefill")


@pytest.mark.parametrize("T,Hq,Hkv,cap,win,p0,kt,qt", [
    (150, 4, 2, 512, 300, 900, 0, F32),          # a wrapped ring under a window
    (260, 2, 1, 640, 350, 1500, 3, BF16),        # the window's first key mid-tile, the ring's seam inside the pass's keys
    (40, 2, 2, 0, 0, 0, 0, F16),                 # one tile
    (100, 2, 1, 0, 0, 28, 3, BF16),              # two tiles
    (130, 2, 1, 0, 0, 62, 0, F32),               # three
    (200, 2, 1, 0, 0, 56, 0, F16),               # four, a pass that starts mid-tile
    (256, 2, 1, 0, 0, 1024, 3, F32),             # whole tiles only
    (257, 2, 1, 0, 100, 777, 0, BF16),           # a row block of one row
])
def test_prefill_tiles_sent_straight_to_lds(ops, tune, T, Hq, Hkv, cap, win, p0, kt, qt):
    """Over 16-bit rows of 128 both forms move their tiles global -> LDS without registers, the 8-wave form into three
    buffers a stream, the 4-wave form into two: passes of one to many tiles (every buffer rotation of either), rings
    with their seam among the pass's keys, windows whose edge falls inside a tile - against the float64 closed form, and
    the two forms bit for bit against each other."""
    D = 128
    n = p0 + T
    if cap:
        k = orc.randn(31, (n, Hkv * D))
        v = orc.randn(32, (n, Hkv * D))
        kc = np.zeros((Hkv, cap, 2 * D), np.uint8)
        vc = np.zeros((Hkv, cap, 2 * D), np.uint8)
        for s0 in range(0, n, 128):
            e = min(n, s0 + 128)
            orc.kv_store(kt, k[s0:e], v[s0:e], Hkv, D, cap, s0, kc, vc, ring=True)
    else:
        cap = n + 3
        kc, vc = make_kv(kt, Hkv, D, cap, n, cfg=2)
    qd, qf = make_q(qt, T, Hq, D, cfg=1)
    tune(TUNE_PREFILL_WAVES, 8)
    got8, _ = gpu_prompt(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    tune(TUNE_PREFILL_WAVES, 4)
    got4, _ = gpu_prompt(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    ref = orc.attn_f64(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(got8, ref, qt, "prefill, tiles straight to LDS", kt=kt)
    assert np.array_equal(got8, got4)


def test_prompt_rows_agree_with_decode_rows(ops):
    """The reference's --prompt-decode check (cli/nextsycl/src/main.rs:869-917): a prompt pass's row t against the
    decode pass at position p0 + t - two kernels, one result within the path's tolerance."""
    T, Hq, Hkv, D, p0 = 64, 8, 2, 128, 200
    cap = p0 + T
    kc, vc = make_kv(0, Hkv, D, cap, cap)
    qd, qf = make_q(F32, T, Hq, D)
    g = ops.gpu
    bufs = (DevBuf.of(g, kc), DevBuf.of(g, vc))
    pr, _ = gpu_prompt(ops, F32, 0, qd, kc, vc, T, Hq, Hkv, D, cap, p0, bufs=bufs)
    for t in (0, 1, 31, 63):
        de, _ = gpu_decode(ops, F32, 0, qd[t:t + 1], kc, vc, 1, Hq, Hkv, D, cap, p0 + t, bufs=bufs)
        mx, rel, _ = orc.compare(pr[t:t + 1], de.astype(np.float64))
        assert mx <= 2e-3 and rel <= 1e-3, (t, mx, rel)


def test_softmax_weights_sum_to_one(ops):
    """V = 1 everywhere -> every output is 1: a row's weights sum to one (to the rounding of the weights to half)."""
    T, Hq, Hkv, D = 400, 4, 1, 128
    kc, vc = make_kv(0, Hkv, D, T, T)
    vc = np.ascontiguousarray(np.broadcast_to(np.array([0x3C00], np.uint16).view(np.uint8), (Hkv, T, D, 2)).reshape(Hkv, T, 2 * D))
    qd, _ = make_q(F32, T, Hq, D)
    got, _ = gpu_prompt(ops, F32, 0, qd, kc, vc, T, Hq, Hkv, D, T, 0)
    assert np.abs(got - 1.0).max() < 5e-4


def test_reference_named_prompt_entry_points(ops):
    T, Hq, Hkv, D, p0 = 70, 8, 2, 128, 10
    cap = p0 + T
    kc, vc = make_kv(0, Hkv, D, cap, cap)
    qd, _ = make_q(F32, T, Hq, D)
    g = ops.gpu
    bufs = (DevBuf.of(g, kc), DevBuf.of(g, vc))
    want, _ = gpu_prompt(ops, F32, 0, qd, kc, vc, T, Hq, Hkv, D, cap, p0, bufs=bufs)
    qb, ob = DevBuf.of(g, qd), DevBuf(g, T * Hq * D * 4)
    k = ops.k
    assert k.mg_attn_prompt_supported(T, Hq, Hkv, D) == 1 and k.mg_attn_prompt_supported(16, Hq, Hkv, D) == 0
    ops.mg_attn_prompt(qb, bufs[0], bufs[1], T, Hq, Hkv, D, cap, p0, 0, ob)
    assert np.array_equal(ob.read(np.float32).reshape(T, -1), want)
    ob.fill(0)
    ops.mg_attn(qb, bufs[0], bufs[1], T, Hq, Hkv, D, cap, p0, 0, True, ob, None)
    assert np.array_equal(ob.read(np.float32).reshape(T, -1), want)
    ob.fill(0)
    ops.q35_attn(qb, Hq * D, bufs[0], bufs[1], T, Hq, Hkv, D, cap, p0, ob, None)
    assert np.array_equal(ob.read(np.float32).reshape(T, -1), want)
    assert k.attn_prompt_t(g.raw, 0, 0, 0, qb.ptr, Hq * D, bufs[0].ptr, bufs[1].ptr, T, Hq, Hkv, 64, cap, p0, 0, 0.0, ob.ptr) == -1
    assert "heads of 128 or 256" in k.api.error()


WIDE = [
    # T, Hq, Hkv, p0, win, kt, qt        heads of 256 (Qwen3.5's), every cache form of the reference's prompt kernel
    (17, 6, 1, 0, 0, 0, F32),
    (200, 12, 2, 333, 0, 0, F32),        # G 6, a later chunk
    (130, 4, 2, 0, 0, 3, BF16),
    (190, 12, 2, 100, 0, 1, F32),        # q8_0 rows (272 bytes)
    (150, 6, 1, 60, 0, 2, F16),          # q4_0 rows (144 bytes)
    (100, 4, 1, 700, 128, 1, F32),       # q8_0 under a window
]


@pytest.mark.parametrize("T,Hq,Hkv,p0,win,kt,qt", WIDE)
def test_prefill_heads_of_256_and_quantized_rows(ops, T, Hq, Hkv, p0, win, kt, qt):
    D = 256
    cap = p0 + T + 3
    kc, vc = make_kv(kt, Hkv, D, cap, p0 + T)
    qd, qf = make_q(qt, T, Hq, D)
    got, _ = gpu_prompt(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    ref = orc.attn_f64(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(got, ref, qt, "prefill, heads of 256", kt=kt)


@pytest.mark.parametrize("T,Hq,Hkv,D,p0", [(90, 12, 2, 256, 40), (300, 16, 2, 128, 500), (1100, 16, 1, 128, 0)])
def test_q35_prompt_kv_entry_point(ops, T, Hq, Hkv, D, p0):
    """ns_q35_attn_prompt_kv as the engine calls it (llm/qwen35/src/engine.rs:1598-1617): float32 rows, D = 256, Hq = 6 Hkv;
    and over heads of 128 (136- / 72-byte rows: the cache form of the 128K q8_0 decode configuration taking a prompt)."""
    cap = p0 + T
    g = ops.gpu
    qd, qf = make_q(F32, T, Hq, D)
    for kt in (0, 1, 2):
        kc, vc = make_kv(kt, Hkv, D, cap, cap)
        ob = DevBuf(g, T * Hq * D * 4); ob.fill(0xFF)
        qb, kb, vb = DevBuf.of(g, qd), DevBuf.of(g, kc), DevBuf.of(g, vc)        # held: a buffer is freed with its object
        rc = ops.k.q35_attn_prompt_kv(g.raw, kt, qb.ptr, Hq * D, kb.ptr, vb.ptr, T, Hq, Hkv, D, cap, p0, ob.ptr)
        assert rc == 0, ops.k.api.error()
        check_close(ob.read(np.float32).reshape(T, -1), orc.attn_f64(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0), F32, "ns_q35_attn_prompt_kv kt %d" % kt)


@pytest.mark.parametrize("T,Hq,Hkv,D,p0,win,kt,qt", [
    (200, 8, 2, 128, 300, 0, 0, F32),
    (200, 8, 2, 128, 300, 0, 3, BF16),           # the bfloat16 rows are widened out of a position-major cache
    (333, 10, 2, 128, 1000, 150, 3, F32),        # under a window: the widened copy starts at the window's first key
    (90, 4, 4, 256, 40, 0, 3, F16),
    (300, 6, 2, 128, 200, 0, 1, F16),
])
def test_prompt_over_a_position_major_cache(ops, T, Hq, Hkv, D, p0, win, kt, qt):
    """Prompt passes over caches laid out [position][key head][row] (MiniMax-M3's layout: kernels/llm/minimaxm3/mm3.h:33-37),
    every cache form the typed entry point takes - a bfloat16 cache's rows are widened to half from that layout too."""
    n = p0 + T
    cap = n + 5
    kc, vc = make_kv(kt, Hkv, D, cap, n, cfg=1, pm=True)
    qd, qf = make_q(qt, T, Hq, D, cfg=2)
    got, _ = gpu_prompt(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win, pm=True)
    ref = orc.attn_f64(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win, pm=True)
    check_close(got, ref, qt, "prompt over a position-major cache", kt=kt)


PACKED = [
    # T, Hq, Hkv, D, p0, win, kt, qt: passes of so few rows that a work-group holds 2 or 4 query heads of its key head
    (17, 8, 2, 128, 5000, 0, 0, F16),           # 4 heads a work-group, key splits
    (32, 16, 2, 128, 300, 0, 0, F32),           # G 8: two work-groups of 4 heads a key head
    (33, 8, 2, 128, 9000, 0, 3, BF16),          # 2 heads a work-group; bfloat16 operands (few rows: not widened)
    (20, 12, 2, 128, 700, 256, 1, F16),         # G 6: 2 heads; a window; q8_0 rows widened
    (64, 6, 1, 128, 2000, 0, 2, F32),           # q4_0 rows of 128 in the kernel's own staging, 2 heads
    (17, 12, 2, 256, 4000, 0, 0, F32),          # heads of 256: 17 rows fill two of four waves
    (5, 8, 2, 256, 1000, 0, 1, F16),            # ... 5 rows: 4 heads a work-group
    (16, 10, 2, 128, 100, 0, 0, F32),           # G 5: five heads to an 8-wave work-group, three waves without rows
    (30, 20, 4, 128, 6000, 0, 3, BF16),         # ... behind key splits, bfloat16
    (40, 14, 2, 128, 900, 0, 0, F16),           # G 7, two waves a head: no divisor fits - one head a work-group
    (9, 14, 2, 256, 900, 0, 0, F16),            # G 7 at heads of 256: seven heads to 8 waves
    (20, 6, 2, 128, 3000, 0, 1, F32),           # G 3: three heads to 4 waves
    (33, 20, 2, 128, 2000, 100, 0, F32),        # G 10, two waves a head: 2 heads (4 waves); a window
    (40, 4, 1, 128, 0, 0, 0, F16),              # no context: the last rows' blocks see few keys
]


@pytest.mark.parametrize("T,Hq,Hkv,D,p0,win,kt,qt", PACKED)
def test_prefill_work_groups_holding_several_heads(ops, T, Hq, Hkv, D, p0, win, kt, qt):
    cap = p0 + T + 3
    kc, vc = make_kv(kt, Hkv, D, cap, p0 + T, cfg=4)
    qd, qf = make_q(qt, T, Hq, D, cfg=2)
    got, _ = gpu_prompt(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    ref = orc.attn_f64(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(got, ref, qt, "prefill, several heads a work-group", kt=kt)


@pytest.mark.parametrize("T,Hq,Hkv,D,p0", [(20, 16, 2, 128, 3000), (64, 8, 2, 128, 500), (100, 4, 2, 128, 9000), (10, 8, 1, 256, 700), (30, 8, 2, 256, 0)])
def test_prefill_8_wave_work_groups_holding_several_heads(ops, tune, T, Hq, Hkv, D, p0):
    """The 8-wave form (knob 2) over passes of few rows: 8, 4 or 2 heads a work-group; the same results as the 4-wave
    form's to the bound (their key splits differ with the heads a work-group holds)."""
    cap = p0 + T + 1
    kc, vc = make_kv(0, Hkv, D, cap, p0 + T, cfg=1)
    qd, qf = make_q(F16, T, Hq, D, cfg=3)
    ref = orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, cap, p0)
    for waves in (8, 4):
        tune(TUNE_PREFILL_WAVES, waves)
        got, _ = gpu_prompt(ops, F16, 0, qd, kc, vc, T, Hq, Hkv, D, cap, p0)
        check_close(got, ref, F16, "prefill, %d waves, several heads a work-group" % waves)


def _own_form_cases():
    """Every case of the tables above over a cache that is not half, as (T, Hq, Hkv, D, p0, win, kt, qt)."""
    out = [(T, Hq, Hkv, 128, p0, win, kt, qt) for T, Hq, Hkv, p0, win, kt, qt in SMALL + QROWS128]
    out += [(T, Hq, Hkv, 256, p0, win, kt, qt) for T, Hq, Hkv, p0, win, kt, qt in WIDE]
    out += SPLIT + _random_cases(32, 20240608)
    return [c for c in out if c[6] != 0]


@pytest.mark.parametrize("T,Hq,Hkv,D,p0,win,kt,qt", _own_form_cases())
def test_prefill_over_the_caches_own_form(ops, tune, T, Hq, Hkv, D, p0, win, kt, qt):
    """A pass over bfloat16, q8_0 or q4_0 rows first widens them to half rows in the library's scratch and runs as a
    pass over a half cache (knob 5 = 2 here: always); a pass of few rows, or one whose context is too long for the scratch
    (knob 5 = 1 here), keeps the rows' own form in the kernel. Both meet the bound; over quantized rows both stage the same halfs (half(q x d), one rounding) and walk the
    keys in the same order, so they agree bit for bit."""
    cap = p0 + T + 7
    kc, vc = make_kv(kt, Hkv, D, cap, p0 + T, cfg=2)
    qd, qf = make_q(qt, T, Hq, D, cfg=1)
    tune(5, 2)
    wide, _ = gpu_prompt(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    tune(5, 1)
    own, _ = gpu_prompt(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win)
    ref = orc.attn_f64(qf, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
    check_close(wide, ref, qt, "prefill, rows widened first", kt=kt)
    # (bfloat16 operands: query rows of another type enter the first product as two bfloat16 numbers - the same bound)
    check_close(own, ref, qt, "prefill, the cache's own form in the kernel", kt=kt)
    if kt in (1, 2) and not (kt == 2 and D == 128):
        assert np.array_equal(np.asarray(wide).view(np.uint8), np.asarray(own).view(np.uint8))
