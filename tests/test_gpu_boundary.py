"""The entry points an engine binds beyond the typed kernels - the drafter's block (not causal), the MiniMax silo's
names, ns_q35_attn_probs, ns_mla_attend, ns_gather_q8_h, longer ns_mla_attend_sel passes - through the C ABI against the
oracle (pinned in tests/test_oracle_boundary.py, tests/test_oracle_attention.py). Attention within max-abs 2e-3 /
relative L2 1e-3 of the float64 closed form; byte formats bit for bit."""
import numpy as np
import pytest

from helpers import check_close, make_kv, make_q
from nextsycl_amd import DevBuf, Error
from nextsycl_amd.attn import F32
from oracle import orc

pytestmark = pytest.mark.gpu


def _ring_caches(Hkv, D, cap, n, seed):
    """Half ring caches [Hkv][cap][D] holding the last `cap` of positions 0 .. n - 1 (slot = position % cap)."""
    k, v = orc.randn(seed, (n, Hkv * D)), orc.randn(seed + 1, (n, Hkv * D))
    kc = np.zeros((Hkv, cap, 2 * D), np.uint8)
    vc = np.zeros((Hkv, cap, 2 * D), np.uint8)
    for s in range(0, n, 64):
        e = min(n, s + 64)
        orc.kv_store(0, k[s:e], v[s:e], Hkv, D, cap, s, kc=kc, vc=vc, ring=True)
    return kc, vc


# the drafter's block as the engine calls it: ns_mg_attn(win = the draft window, causal = 0). The last four shapes are ones
# whose rows' own split sizes differ (a 128-multiple is crossed inside the block): the pass must still be one launch
# cut by its first row's key count
BLOCKS = [(2, 8, 2, 128, 5000, 0), (8, 16, 4, 128, 3000, 2048), (16, 8, 2, 128, 9000, 4096), (16, 32, 8, 128, 20000, 8192),
          (8, 32, 8, 128, 8190, 8192), (5, 16, 8, 256, 4094, 4096), (16, 32, 16, 128, 4090, 4096), (3, 32, 16, 256, 2046, 2048),
          (4, 8, 2, 128, 100, 0), (16, 4, 1, 128, 0, 0)]


@pytest.mark.parametrize("T,Hq,Hkv,D,p0,win", BLOCKS)
def test_block_that_is_not_causal(ops, T, Hq, Hkv, D, p0, win):
    g = ops.gpu
    cap = p0 + T if win == 0 else win + T - 1 + 3
    if win == 0:
        kc, vc = make_kv(0, Hkv, D, cap, p0 + T, cfg=T)
    else:
        kc, vc = _ring_caches(Hkv, D, cap, p0 + T, 100 + T)
    qd, qf = make_q(F32, T, Hq, D, cfg=p0 % 7)
    ref = orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, cap, p0, win=win, causal=False)
    qb, kb, vb = DevBuf.of(g, qd), DevBuf.of(g, kc), DevBuf.of(g, vc)
    ob = DevBuf(g, T * Hq * D * 4); ob.fill(0xFF)
    sc = DevBuf(g, 4 * ops.k.mg_attn_scratch(T, Hq, Hkv, D, p0, win, 0))
    ops.mg_attn(qb, kb, vb, T, Hq, Hkv, D, cap, p0, win, False, ob, sc)
    got = ob.read(np.float32).reshape(T, -1)
    check_close(got, ref, F32, "ns_mg_attn, not causal")
    # the silo's name for it: the same launch, the same bits
    ob2 = DevBuf(g, T * Hq * D * 4); ob2.fill(0xFF)
    sc2 = DevBuf(g, 4 * ops.k.mg_attn_block_scratch(T, Hq, Hkv, D, p0, win))
    ops.mg_attn_block(qb, kb, vb, T, Hq, Hkv, D, cap, p0, win, ob2, sc2)
    assert np.array_equal(ob2.read(np.float32).reshape(T, -1), got)
    # and it differs from the causal pass wherever a row has later rows behind it
    if T > 1:
        assert np.abs(orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, cap, p0, win=win)[0] - ref[0]).max() > 1e-4


@pytest.mark.parametrize("T,Hq,Hkv,D,p0,win", [(40, 8, 2, 128, 700, 0), (70, 4, 1, 128, 3000, 512), (33, 4, 2, 256, 300, 0), (300, 4, 2, 128, 0, 0)])
def test_long_block_that_is_not_causal(ops, T, Hq, Hkv, D, p0, win):
    """More than 16 rows: the prompt kernel with every row ending at the pass's last key (kernels/llm/museglimmer/mg.cpp:58,
    227-229 runs any row count that way)."""
    g = ops.gpu
    cap = p0 + T if win == 0 else win + T - 1 + 5
    kc, vc = make_kv(0, Hkv, D, cap, p0 + T, cfg=1) if win == 0 else _ring_caches(Hkv, D, cap, p0 + T, 300)
    qd, qf = make_q(F32, T, Hq, D, cfg=2)
    ob = DevBuf(g, T * Hq * D * 4); ob.fill(0xFF)
    ops.mg_attn(DevBuf.of(g, qd), DevBuf.of(g, kc), DevBuf.of(g, vc), T, Hq, Hkv, D, cap, p0, win, False, ob, None)
    check_close(ob.read(np.float32).reshape(T, -1), orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, cap, p0, win=win, causal=False), F32,
                "ns_mg_attn, not causal, prompt kernel")


def _mm3_inputs(T, H, G, pos0, seed=0):
    n = pos0 + T
    q = orc.randn(60 + seed, (T, H * 128))
    kc, _ = orc.randn_f16(61 + seed, (n, G, 128)); vc, _ = orc.randn_f16(62 + seed, (n, G, 128))
    return n, q, kc, vc


@pytest.mark.parametrize("T,H,G,pos0", [(1, 32, 2, 4000), (4, 16, 1, 700), (40, 32, 2, 900)])
def test_mm3s_names_are_the_shared_kernels(ops, T, H, G, pos0):
    """ns_mm3s_attend / _x / _split / _x_split give ns_llm_minimaxm3_attend's bits (one kernel family behind every name),
    dense and with block lists; the split forms go through the caller's `part`."""
    g = ops.gpu
    n, q, kc, vc = _mm3_inputs(T, H, G, pos0)
    scale = 1.0 / np.sqrt(128.0)
    assert ops.k.mm3s_attend_supported(H, G, 128) == 1 and ops.k.mm3s_attend_supported(H, G, 64) == 0
    qb, kb, vb = DevBuf.of(g, q), DevBuf.of(g, kc), DevBuf.of(g, vc)
    nblk = (n + 127) // 128
    K = min(6, nblk)
    rng = np.random.default_rng(3)
    sel = np.stack([np.stack([rng.permutation(nblk)[:K] for _ in range(G)]) for _ in range(T)]).astype(np.int32)
    sel[-1, -1, 0] = nblk - 1
    for lists in (None, sel):
        sb = DevBuf.of(g, lists) if lists is not None else None
        kk = K if lists is not None else 0
        base = DevBuf(g, T * H * 128 * 4); base.fill(0xFF)
        ops.minimaxm3_attend(qb, kb, vb, base, T, H, G, pos0, scale, sel=sb, K=kk)
        want = base.read(np.float32)
        close_to = orc.mm3_attend(q, kc, vc, T, H, G, pos0, scale, sel=lists, K=kk)
        check_close(want.reshape(T, -1), close_to.astype(np.float64), F32, "minimaxm3_attend")
        S = kk if lists is not None else nblk
        for form in ("", "x", "split", "x_split"):
            ob = DevBuf(g, T * H * 128 * 4); ob.fill(0xFF)
            part = DevBuf(g, T * G * S * 16 * 130 * 4) if "split" in form else None
            if part is not None:
                part.fill(0xFF)
            # the matrix-unit names take any scale that is not positive as 1 / sqrt(128)
            ops.mm3s_attend(form, qb, kb, vb, ob, T, H, G, pos0, 0.0 if form.startswith("x") else scale, sel=sb, K=kk, S=S, part=part)
            assert np.array_equal(ob.read(np.float32), want), (form, lists is not None)
            if part is not None and T <= 16 and H == 16 * G:
                assert not np.all(part.read(np.uint8) == 0xFF), "the caller's part was not used"


@pytest.mark.parametrize("T,H,G,pos0,w0", [(8, 32, 2, 3000, 1234), (16, 16, 1, 5000, 0), (4, 16, 1, 227 - 3, 100), (24, 32, 2, 2000, 777)])
def test_mm3s_attend_block(ops, T, H, G, pos0, w0):
    """A draft block: every row sees keys w0 .. pos0 + T - 1. (The third shape: 128 keys that straddle a 128-key boundary -
    one split more than the caller's S = 1 holds, so the partials go through the library's own memory.)"""
    g = ops.gpu
    n, q, kc, vc = _mm3_inputs(T, H, G, pos0, seed=5)
    S = (n - w0 + 127) // 128
    part = DevBuf(g, T * G * S * 16 * 130 * 4)
    ob = DevBuf(g, T * H * 128 * 4); ob.fill(0xFF)
    ops.mm3s_attend("block", DevBuf.of(g, q), DevBuf.of(g, kc), DevBuf.of(g, vc), ob, T, H, G, pos0, 0.0, S=S, part=part, w0=w0)
    ref = orc.attn_f64_block(q, kc.view(np.uint8), vc.view(np.uint8), 0, T, H, G, 128, n, pos0, w0, pm=True)
    check_close(ob.read(np.float32).reshape(T, -1), ref, F32, "ns_mm3s_attend_block")


@pytest.mark.parametrize("kt,Hq,Hkv,D,cap,n", [(0, 12, 2, 256, 3000, 2777), (1, 12, 2, 256, 900, 900), (2, 6, 1, 256, 500, 333),
                                               (0, 32, 8, 128, 1500, 1499), (1, 8, 8, 128, 70, 1),
                                               (3, 8, 2, 128, 41000, 40001), (0, 6, 1, 256, 17000, 16999)])   # a head's statistics over 4 and 2 key slices
def test_q35_attn_probs(ops, kt, Hq, Hkv, D, cap, n):
    g = ops.gpu
    k = orc.randn(70 + kt, (cap, Hkv * D))
    kc, _ = orc.kv_store(kt, k, k, Hkv, D, cap, 0)
    q = orc.randn(71, (Hq, D), 0.6)
    base = np.linspace(0.0, 0.5, n).astype(np.float32)
    qb, kb = DevBuf.of(g, q), DevBuf.of(g, kc)
    for mode in (0, 1):
        ob = DevBuf.of(g, base)
        sc = DevBuf(g, 2 * Hq * 4)
        ops.q35_attn_probs(kt, qb, kb, Hq, Hkv, D, cap, n, mode, sc, ob)
        got = ob.read(np.float32)
        want = orc.attn_probs(kt, q, kc, Hq, Hkv, D, cap, n, mode, out=base)
        # float32 softmax weights summed in another order: a few ulps of the largest weight
        assert np.abs(got - want).max() <= 2e-6 + 1e-5 * np.abs(want - base).max(), (mode, np.abs(got - want).max())
        if mode == 0:
            assert abs(float((got.astype(np.float64) - base).sum()) - 1.0) < 1e-4


def test_glm_dense_over_a_float32_cache(ops):
    g = ops.gpu
    L, scale = 512, 0.044
    for T, H, pos0 in ((1, 64, 2047), (5, 16, 300), (40, 8, 100)):
        n = pos0 + T
        qa, c = orc.randn(80, (T, H * L), 0.3), orc.randn(81, (n, L))
        u = DevBuf(g, T * H * L * 4); u.fill(0xFF)
        ops.mla_attend_f32(DevBuf.of(g, qa), DevBuf.of(g, c), u, T, H, L, pos0, scale)
        want = orc.glm_mla_attend_f32(qa, c, T, H, L, pos0, scale).reshape(T, H * L)
        check_close(u.read(np.float32).reshape(T, H * L), want.astype(np.float64), F32, "ns_mla_attend")


def test_gather_q8_rows_as_half(ops):
    g = ops.gpu
    L, rows, n = 512, 300, 1000
    y = orc.glm_to_q8row(orc.randn(90, (rows, L), 2.0), L)
    idx = np.random.default_rng(1).integers(0, rows, n).astype(np.int32)
    out = DevBuf(g, n * L * 2); out.fill(0xFF)
    ops.gather_q8_h(DevBuf.of(g, y), rows, DevBuf.of(g, idx), out, n, L)
    assert np.array_equal(out.read(np.uint16).reshape(n, L), orc.glm_gather_q8_h(y, idx, L))


@pytest.mark.parametrize("q8", [False, True])
def test_glm_cell_pools_of_a_long_pass(ops, q8):
    """More rows than one pass of the selection kernel takes (16): queued pass after pass, each row with its own list."""
    g = ops.gpu
    T, H, L, pos0, K, scale = 40, 16, 512, 3000, 32, 0.044
    n = pos0 + T
    qa = orc.randn(91, (T, H * L), 0.3)
    x = orc.randn(92, (n, L))
    rows = orc.glm_to_q8row(x, L) if q8 else orc.f2h(x).view(np.uint8).reshape(n, 2 * L)
    rng = np.random.default_rng(9)
    npool = (pos0 + 1) // 4
    sel = np.stack([rng.permutation(npool)[:K] for _ in range(T)]).astype(np.int32)
    cnt = rng.integers(0, K + 1, T).astype(np.int32)
    u = DevBuf(g, T * H * L * 4); u.fill(0xFF)
    ops.mla_attend(DevBuf.of(g, qa), DevBuf.of(g, rows), u, T, H, L, pos0, scale, q8=q8, sel=DevBuf.of(g, sel), sel_cnt=DevBuf.of(g, cnt), K=K)
    want = orc.glm_mla_attend_sel(qa, rows, q8, T, H, L, pos0, scale, sel, cnt, K)
    check_close(u.read(np.float32).reshape(T, H * L), want.reshape(T, H * L).astype(np.float64), F32, "ns_mla_attend_sel, 40 rows")


@pytest.mark.parametrize("q8", [False, True])
def test_glm_cell_pools_at_100k_tokens(ops, q8):
    """Selection lists over a 100K-token latent cache: 4 rows x 64 heads, 512 pools (2048 cells) a row picked from the whole
    context, against the reference-order restatement."""
    g = ops.gpu
    T, H, L, pos0, K, scale = 4, 64, 512, 100000, 512, 0.044
    n = pos0 + T
    qa = orc.randn(93, (T, H * L), 0.3)
    x = orc.randn(94, (n, L))
    rows = orc.glm_to_q8row(x, L) if q8 else orc.f2h(x).view(np.uint8).reshape(n, 2 * L)
    rng = np.random.default_rng(10)
    npool = (pos0 + 1) // 4
    sel = np.stack([rng.choice(npool, K, replace=False) for _ in range(T)]).astype(np.int32)
    cnt = np.array([K, K - 1, 7, K], np.int32)
    u = DevBuf(g, T * H * L * 4); u.fill(0xFF)
    ops.mla_attend(DevBuf.of(g, qa), DevBuf.of(g, rows), u, T, H, L, pos0, scale, q8=q8, sel=DevBuf.of(g, sel), sel_cnt=DevBuf.of(g, cnt), K=K)
    want = orc.glm_mla_attend_sel(qa, rows, q8, T, H, L, pos0, scale, sel, cnt, K)
    check_close(u.read(np.float32).reshape(T, H * L), want.reshape(T, H * L).astype(np.float64), F32, "ns_mla_attend_sel at 100K tokens")


@pytest.mark.parametrize("T,H,pos0", [(1, 16, 700), (3, 128, 2000), (16, 8, 5), (37, 8, 300)])
def test_ds2_mla_decode_with_q6k_weights(ops, T, H, pos0):
    """ns_ds2_mla_decode_q6k: kv_b read as the file stores it (Q6_K rows), against the float64 chain over the widened rows."""
    from test_oracle_boundary import random_q6k_rows
    g = ops.gpu
    n = pos0 + T
    kvb = random_q6k_rows(31, H * 256).reshape(H, 256, 420)
    cache = orc.f2h(orc.randn(32, (n, 576), 0.5))
    q = orc.randn(33, (T, H, 192))
    scale = 1.0 / np.sqrt(192.0)
    out = DevBuf(g, T * H * 128 * 4); out.fill(0xFF)
    ops.mla_decode_q6k(DevBuf.of(g, q), DevBuf.of(g, kvb), DevBuf.of(g, cache), out, T, H, pos0, scale)
    w = orc.q6k_rows512(kvb).reshape(H, 256, 512).astype(np.float64)
    qa64 = np.concatenate([np.einsum("hic,thi->thc", w[:, :128], q[:, :, :128].astype(np.float64)), q[:, :, 128:]], axis=2)
    u64 = orc.mla_f64(qa64.astype(np.float32), cache, T, H, pos0, scale)
    want = np.einsum("hvc,thc->thv", w[:, 128:], u64)
    got = out.read(np.float32).reshape(T, H * 128)
    # the result is small (weights of 1e-3 x 6-bit values): the bar relative to its own size
    mx, rel, _ = orc.compare(got, want.reshape(T, H * 128))
    assert rel <= 1e-3 and mx <= 2e-3 * max(1.0, np.abs(want).max()), (mx, rel)
    # the restated chain agrees with the float64 one as well
    qa = orc.mla_absorb_q6k(q, kvb, T, H)
    ref = orc.mla_vb_q6k(orc.mla_decode_u(qa, cache, T, H, pos0, scale), kvb, T, H)
    assert orc.compare(ref.reshape(T, H * 128), want.reshape(T, H * 128))[1] <= 1e-4


def test_glm_latent_width_256(ops):
    """The reference's other latent width (kernels/llm/glm5next/glm.cpp:1257): a half cache dense and with cell pools, a
    float32 cache dense - against the reference-order restatement at L = 256 (an instance of the latent kernel of its own
    width: no length is refused)."""
    g = ops.gpu
    L, scale = 256, 0.0625
    for T, H, pos0, K in ((1, 64, 2000, 0), (5, 16, 300, 0), (20, 8, 3000, 24), (3, 32, 20000, 128)):
        n = pos0 + T
        qa, x = orc.randn(95, (T, H * L), 0.3), orc.randn(96, (n, L))
        rows = orc.f2h(x).view(np.uint8).reshape(n, 2 * L)
        rng = np.random.default_rng(11)
        sel = cnt = None
        if K:
            npool = (pos0 + 1) // 4
            sel = np.stack([rng.permutation(npool)[:K] for _ in range(T)]).astype(np.int32)
            cnt = rng.integers(0, K + 1, T).astype(np.int32)
        u = DevBuf(g, T * H * L * 4); u.fill(0xFF)
        ops.mla_attend(DevBuf.of(g, qa), DevBuf.of(g, rows), u, T, H, L, pos0, scale, sel=DevBuf.of(g, sel) if K else None,
                       sel_cnt=DevBuf.of(g, cnt) if K else None, K=K)
        want = orc.glm_mla_attend_sel(qa, rows, False, T, H, L, pos0, scale, sel, cnt, K) if K else orc.glm_mla_attend(qa, rows, False, T, H, L, pos0, scale)
        check_close(u.read(np.float32).reshape(T, H * L), want.reshape(T, H * L).astype(np.float64), F32, "ns_mla_attend_sel at L = 256, %d rows" % T)
        if not K and pos0 < 3000:
            u.fill(0xFF)
            ops.mla_attend_f32(DevBuf.of(g, qa), DevBuf.of(g, x), u, T, H, L, pos0, scale)
            want = orc.glm_mla_attend_f32(qa, x, T, H, L, pos0, scale).reshape(T, H * L)
            check_close(u.read(np.float32).reshape(T, H * L), want.astype(np.float64), F32, "ns_mla_attend at L = 256")
    # a length no scratch bounds: 100,000 cells, a row with cell pools (what the engine passes past 2,560 tokens) against the
    # float64 closed form over the row's listed cells
    T, H, pos0, K = 2, 16, 100000, 64
    n = pos0 + T
    qa, x = orc.randn(97, (T, H * L), 0.3), orc.randn(98, (n, L), 0.5)
    rows = orc.f2h(x).view(np.uint8).reshape(n, 2 * L)
    rng = np.random.default_rng(12)
    sel = np.stack([np.sort(rng.permutation((pos0 + 1) // 4)[:K]) for _ in range(T)]).astype(np.int32)
    cnt = np.array([K, K // 2], np.int32)
    u = DevBuf(g, T * H * L * 4); u.fill(0xFF)
    ops.mla_attend(DevBuf.of(g, qa), DevBuf.of(g, rows), u, T, H, L, pos0, scale, sel=DevBuf.of(g, sel), sel_cnt=DevBuf.of(g, cnt), K=K)
    want = orc.glm_mla_attend_sel(qa, rows, False, T, H, L, pos0, scale, sel, cnt, K)
    check_close(u.read(np.float32).reshape(T, H * L), want.reshape(T, H * L).astype(np.float64), F32, "ns_mla_attend_sel at L = 256, 100,000 cells")


# ricursive's engine (ns_rc_*: a ring of R rows a head, a window W, 10 query heads a key head among its ratios) and
# nemotron-h's attention layers (ns_nh_*: plain causal, 8 query heads a key head)
RC = [
    # T, Hq, Hkv, R, W, p0
    (1, 10, 1, 4096, 0, 3000),          # one decode row, all keys, the cache not yet a ring
    (1, 20, 2, 1024, 1000, 5000),       # a wrapped ring under a window
    (8, 10, 1, 600, 512, 2047),         # verify rows; the ring's seam inside the window
    (16, 12, 2, 2048, 0, 100),          # 6 query heads a key head
    (40, 10, 1, 700, 600, 1500),        # a prompt chunk through the ring
    (300, 8, 4, 400, 64, 900),          # more rows than the window: R >= W + T - 1
]


@pytest.mark.parametrize("T,Hq,Hkv,R,W,p0", RC)
def test_ricursive_entry_points(ops, T, Hq, Hkv, R, W, p0):
    """ns_rc_kv_store writes the ring the oracle's store writes, byte for byte; ns_rc_attn over it against the float64
    closed form (kernels/llm/ricursive/rc.cpp:182-225)."""
    D = 128
    g = ops.gpu
    n = p0 + T
    k, v = orc.randn(41, (n, Hkv * D)), orc.randn(42, (n, Hkv * D))
    kc = np.zeros((Hkv, R, 2 * D), np.uint8)
    vc = np.zeros((Hkv, R, 2 * D), np.uint8)
    kcb, vcb = DevBuf.of(g, kc), DevBuf.of(g, vc)
    step = min(R, 96)
    for s in range(0, n, step):
        e = min(n, s + step)
        orc.kv_store(0, k[s:e], v[s:e], Hkv, D, R, s, kc=kc, vc=vc, ring=True)
        ops.rc_kv_store(DevBuf.of(g, k[s:e]), Hkv * D, DevBuf.of(g, v[s:e]), Hkv * D, e - s, Hkv, D, R, s, kcb, vcb)
    assert np.array_equal(kcb.read(np.uint8).reshape(kc.shape), kc) and np.array_equal(vcb.read(np.uint8).reshape(vc.shape), vc)
    qd, qf = make_q(F32, T, Hq, D)
    ob = DevBuf(g, T * Hq * D * 4)
    ob.fill(0xFF)
    sc = DevBuf(g, max(4, 4 * ops.k.rc_attn_scratch(T, Hq, Hkv, D, W, p0)))
    ops.rc_attn(DevBuf.of(g, qd), Hq * D, kcb, vcb, T, Hq, Hkv, D, R, W, p0, ob, sc)
    got = ob.read(np.float32).reshape(T, Hq * D)
    check_close(got, orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, R, p0, win=W), F32, "ns_rc_attn vs float64 closed form")


@pytest.mark.parametrize("T,Hkv,R,W,p0", [(1, 2, 4096, 0, 3000), (4, 1, 512, 500, 2045), (16, 2, 300, 256, 1000), (40, 1, 700, 512, 5000),
                                          (300, 2, 900, 0, 600)])
def test_ricursive_silo_names(ops, T, Hkv, R, W, p0):
    """ns_rc_flash_decode / ns_rc_flash_prompt (kernels/llm/ricursive/silo/attn.cpp:282-360) over a ring written by
    ns_rc_kv_store: the float64 closed form, and the very bits of ns_rc_attn, whose passes they are."""
    D, Hq = 128, 10 * Hkv
    g = ops.gpu
    n = p0 + T
    k, v = orc.randn(43, (n, Hkv * D)), orc.randn(44, (n, Hkv * D))
    kc = np.zeros((Hkv, R, 2 * D), np.uint8)
    vc = np.zeros((Hkv, R, 2 * D), np.uint8)
    for s in range(0, n, R):
        orc.kv_store(0, k[s:min(n, s + R)], v[s:min(n, s + R)], Hkv, D, R, s, kc=kc, vc=vc, ring=True)
    kcb, vcb = DevBuf.of(g, kc), DevBuf.of(g, vc)
    qd, qf = make_q(F32, T, Hq, D)
    qb = DevBuf.of(g, qd)
    assert ops.k.rc_flash_decode_supported(T, Hq, Hkv, D) == (T <= 16) and ops.k.rc_flash_prompt_supported(T, Hq, Hkv, D) == (T > 16)
    assert not ops.k.rc_flash_decode_supported(1, 8 * Hkv, Hkv, D) and not ops.k.rc_flash_prompt_supported(64, Hq, Hkv, 256)
    ob = DevBuf(g, T * Hq * D * 4)
    ob.fill(0xFF)
    sc = DevBuf(g, max(4, 4 * ops.k.rc_flash_decode_scratch(T, Hq, Hkv, D, p0, W))) if T <= 16 else None
    ops.rc_flash(qb, kcb, vcb, T, Hq, Hkv, D, R, p0, W, ob, sc)
    got = ob.read(np.float32).reshape(T, Hq * D)
    check_close(got, orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, R, p0, win=W), F32, "ricursive's silo names vs float64 closed form")
    ob2 = DevBuf(g, T * Hq * D * 4)
    sc2 = DevBuf(g, max(4, 4 * ops.k.rc_attn_scratch(T, Hq, Hkv, D, W, p0)))
    ops.rc_attn(qb, Hq * D, kcb, vcb, T, Hq, Hkv, D, R, W, p0, ob2, sc2)
    assert np.array_equal(ob2.read(np.float32).view(np.uint32), got.reshape(-1).view(np.uint32))


def test_ricursive_entry_points_refuse_what_the_reference_refuses(ops):
    g = ops.gpu
    D, Hkv = 128, 1
    kcb = DevBuf(g, Hkv * 64 * 2 * D)
    q, out = DevBuf(g, 16 * 10 * D * 4), DevBuf(g, 16 * 10 * D * 4)
    sc = DevBuf(g, 1 << 20)
    with pytest.raises(Error, match="the ring is smaller than the window and the rows"):
        ops.rc_attn(q, 10 * D, kcb, kcb, 4, 10, Hkv, D, 64, 64, 100, out, sc)
    with pytest.raises(Error, match="past the cache's capacity"):
        ops.rc_attn(q, 10 * D, kcb, kcb, 4, 10, Hkv, D, 64, 0, 61, out, sc)
    with pytest.raises(Error, match="1, 2, 4, 6, 8 or 10 query heads a key head"):
        ops.rc_attn(q, 5 * D, kcb, kcb, 1, 5, Hkv, D, 64, 0, 10, out, sc)
    with pytest.raises(Error, match="more rows than the ring holds"):
        ops.rc_kv_store(DevBuf(g, 65 * D * 4), D, DevBuf(g, 65 * D * 4), D, 65, Hkv, D, 64, 0, kcb, kcb)
    with pytest.raises(Error, match="query heads a multiple of 8 a key head"):
        ops.nh_attn(q, 10 * D, kcb, kcb, 1, 10, Hkv, D, 64, 3, out, sc)
    with pytest.raises(Error, match="past the cache's capacity"):
        ops.nh_attn(q, 8 * D, kcb, kcb, 2, 8, Hkv, D, 64, 63, out, sc)
    ops.rc_attn(q, 10 * D, kcb, kcb, 0, 10, Hkv, D, 64, 0, 1000, out, None)      # no rows: nothing is checked
    with pytest.raises(Error, match="1..16 rows, heads of 128, 10 query heads a key head"):
        ops.rc_flash(q, kcb, kcb, 4, 8, Hkv, D, 64, 10, 0, out, sc)
    with pytest.raises(Error, match="ns_rc_flash_decode: no scratch"):
        ops.rc_flash(q, kcb, kcb, 4, 10, Hkv, D, 64, 10, 0, out, None)
    big_q, big_out = DevBuf(g, 40 * 10 * D * 4), DevBuf(g, 40 * 10 * D * 4)
    with pytest.raises(Error, match="the cache's ring is shorter than the window and the pass"):
        ops.rc_flash(big_q, kcb, kcb, 40, 10, Hkv, D, 64, 100, 32, big_out)


@pytest.mark.parametrize("T,Hq,Hkv,p0", [(1, 32, 4, 5000), (4, 16, 2, 2046), (16, 8, 1, 77), (200, 16, 2, 300)])
def test_nemotronh_entry_points(ops, T, Hq, Hkv, p0):
    """ns_nh_kv_store / ns_nh_attn (kernels/llm/nemotronh/nh.cpp:551-588): the store byte for byte, the attention against
    the float64 closed form, and - up to 16 rows - the very bits of ns_q35_attn, whose pass it is."""
    D = 128
    g = ops.gpu
    cap = p0 + T + 3
    k, v = orc.randn(51, (p0 + T, Hkv * D)), orc.randn(52, (p0 + T, Hkv * D))
    kc, vc = orc.kv_store(0, k, v, Hkv, D, cap, 0)
    kcb, vcb = DevBuf(g, kc.nbytes), DevBuf(g, vc.nbytes)
    kcb.fill(0)
    vcb.fill(0)
    # rows of a wider buffer (strides of their own), in two calls
    wide_k, wide_v = np.zeros((p0 + T, Hkv * D + 32), np.float32), np.zeros((p0 + T, Hkv * D + 64), np.float32)
    wide_k[:, :Hkv * D], wide_v[:, :Hkv * D] = k, v
    h = (p0 + T) // 2
    for s, e in ((0, h), (h, p0 + T)):
        if e > s:
            ops.nh_kv_store(DevBuf.of(g, wide_k[s:e]), Hkv * D + 32, DevBuf.of(g, wide_v[s:e]), Hkv * D + 64, e - s, Hkv, D, cap, s, kcb, vcb)
    assert np.array_equal(kcb.read(np.uint8).reshape(kc.shape), kc) and np.array_equal(vcb.read(np.uint8).reshape(vc.shape), vc)
    qd, qf = make_q(F32, T, Hq, D)
    qb, ob = DevBuf.of(g, qd), DevBuf(g, T * Hq * D * 4)
    ob.fill(0xFF)
    sc = DevBuf(g, max(4, 4 * ops.k.nh_attn_scratch(T, Hq, Hkv, D, p0)))
    ops.nh_attn(qb, Hq * D, kcb, vcb, T, Hq, Hkv, D, cap, p0, ob, sc)
    got = ob.read(np.float32).reshape(T, Hq * D)
    check_close(got, orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, cap, p0), F32, "ns_nh_attn vs float64 closed form")
    ob2 = DevBuf(g, T * Hq * D * 4)
    sc2 = DevBuf(g, max(4, 4 * ops.k.q35_attn_scratch(T, Hq, Hkv, D, p0)))
    ops.q35_attn(qb, Hq * D, kcb, vcb, T, Hq, Hkv, D, cap, p0, ob2, sc2)
    assert np.array_equal(ob2.read(np.float32).reshape(T, Hq * D).view(np.uint32), got.view(np.uint32))


@pytest.mark.parametrize("rope", [0, 1])
def test_ricursive_norm_and_rotary(ops, rope):
    """ns_rc_qk_norm_rope (kernels/llm/ricursive/rc.cpp:148-181) is ns_q35_qk_norm_rope turned over all D features, or
    over none: the same bits, and the oracle's restatement within the path's tolerance."""
    T, H, D, p0, theta, eps = 9, 10, 128, 777, 1.0e6, 1.0e-6
    g = ops.gpu
    x = orc.randn(61, (T, H * D))
    w = (1.0 + 0.1 * orc.randn(62, (D,))).astype(np.float32)
    xb, wb = DevBuf.of(g, x), DevBuf.of(g, w)
    a, b = DevBuf(g, x.nbytes), DevBuf(g, x.nbytes)
    ops.ok(ops.k.rc_qk_norm_rope(ops.raw(), xb.ptr, H * D, D, a.ptr, H * D, T, H, D, wb.ptr, eps, rope, theta, p0), "ns_rc_qk_norm_rope")
    ops.ok(ops.k.q35_qk_norm_rope(ops.raw(), xb.ptr, H * D, D, b.ptr, H * D, T, H, D, wb.ptr, eps, D if rope else 0, theta, p0), "ns_q35_qk_norm_rope")
    got = a.read(np.float32)
    assert np.array_equal(got.view(np.uint32), b.read(np.float32).view(np.uint32))
    ref = orc.q35_norm_rope(x.reshape(T, H, D), T, H, D, w, eps, D if rope else 0, theta, p0)
    # (the angle's argument reduction: an error of about pos * 2^-23 radians, as for the qwen35 entry points)
    assert np.abs(got.reshape(ref.shape) - ref).max() <= (4 * (1 + p0 + T) * 2.0 ** -23 + 2e-6) * float(np.abs(ref).max())
