"""Sparse selection on the GPU: MiniMax-M3's block lists and indexer, GLM's cell pools - against the oracle (pinned in
tests/test_oracle_sparse.py). Attention within max-abs 2e-3 / relative L2 1e-3 of the oracle's float32 result; the
selection itself (comparisons only) bit for bit."""
import numpy as np
import pytest

from nextsycl_amd import DevBuf, Error
from oracle import orc

pytestmark = pytest.mark.gpu


def close(got, want):
    err = np.abs(got - want).max()
    rel = np.linalg.norm((got - want).ravel()) / max(np.linalg.norm(want.ravel()), 1e-30)
    assert err <= 2e-3 and rel <= 1e-3, (err, rel)


@pytest.mark.parametrize("T,H,G,pos0,K", [(1, 8, 2, 2000, 6), (3, 64, 4, 5000, 16), (2, 16, 1, 300, 4)])
def test_minimaxm3_block_lists(ops, T, H, G, pos0, K):
    g = ops.gpu
    n = pos0 + T
    nblk = (n + 127) // 128
    q = orc.randn(41, (T, H * 128))
    kc, _ = orc.randn_f16(42, (n, G, 128)); vc, _ = orc.randn_f16(43, (n, G, 128))
    rng = np.random.default_rng(5)
    sel = np.stack([np.stack([rng.permutation(nblk)[:K] if K <= nblk else np.r_[rng.permutation(nblk), [-1] * (K - nblk)] for _ in range(G)])
                    for _ in range(T)]).astype(np.int32)
    sel[0, 0, 1] = -1                                   # a hole
    sel[-1, -1, 0] = nblk - 1                           # the block the row's own position cuts
    scale = 0.0884
    out = DevBuf(g, T * H * 128 * 4); out.fill(0xFF)
    ops.minimaxm3_attend(DevBuf.of(g, q), DevBuf.of(g, kc), DevBuf.of(g, vc), out, T, H, G, pos0, scale, sel=DevBuf.of(g, sel), K=K)
    want = orc.mm3_attend(q, kc, vc, T, H, G, pos0, scale, sel=sel, K=K)
    close(out.read(np.float32).reshape(T, H * 128), want)
    # every block listed in order = the dense pass
    allb = np.tile(np.arange(nblk, dtype=np.int32), (T, G, 1))
    out2 = DevBuf(g, T * H * 128 * 4)
    ops.minimaxm3_attend(DevBuf.of(g, q), DevBuf.of(g, kc), DevBuf.of(g, vc), out2, T, H, G, pos0, scale, sel=DevBuf.of(g, allb), K=nblk)
    close(out2.read(np.float32).reshape(T, H * 128), orc.mm3_attend(q, kc, vc, T, H, G, pos0, scale))
    # nothing listed: zeros
    none = np.full((T, G, 2), -1, np.int32)
    ops.minimaxm3_attend(DevBuf.of(g, q), DevBuf.of(g, kc), DevBuf.of(g, vc), out2, T, H, G, pos0, scale, sel=DevBuf.of(g, none), K=2)
    assert not out2.read(np.float32).any()


@pytest.mark.parametrize("T,H,G,pos0,K", [(40, 32, 2, 3000, 5), (300, 64, 4, 700, 16), (8200, 64, 4, 1000, 2)])
def test_minimaxm3_block_lists_of_a_prompt(ops, tune, T, H, G, pos0, K):
    """A prompt pass with block lists: every (row, key group) is a unit of one launch, the rows' keys are cut only while
    the units are few, and a pass whose partials outgrow the library's scratch (the last case: 8200 rows x 64 heads with
    256 MiB of it to plan with) goes in several launches. Sampled rows against the oracle's one-row pass at their positions."""
    g = ops.gpu
    if T > 8000:
        tune(6, 256)
    n = pos0 + T
    q = orc.randn(51, (T, H * 128))
    kc, _ = orc.randn_f16(52, (n, G, 128)); vc, _ = orc.randn_f16(53, (n, G, 128))
    rng = np.random.default_rng(9)
    sel = np.full((T, G, K), -1, np.int32)
    for t in range(T):
        nb = (pos0 + t) // 128 + 1                                    # blocks the row can see, its own included
        for gi in range(G):
            pick = rng.permutation(nb)[:K]
            sel[t, gi, :len(pick)] = pick
    sel[T // 2, 0, 0] = -1                                            # a hole
    out = DevBuf(g, T * H * 128 * 4); out.fill(0xFF)
    ops.minimaxm3_attend(DevBuf.of(g, q), DevBuf.of(g, kc), DevBuf.of(g, vc), out, T, H, G, pos0, 0.0884, sel=DevBuf.of(g, sel), K=K)
    got = out.read(np.float32).reshape(T, H * 128)
    assert np.isfinite(got).all()
    rows = sorted(set([0, 1, T // 2, T - 2, T - 1] + [int(t) for t in rng.integers(0, T, 12)]))
    for t in rows:
        want = orc.mm3_attend(q[t:t + 1], kc[:pos0 + t + 1], vc[:pos0 + t + 1], 1, H, G, pos0 + t, 0.0884, sel=sel[t:t + 1], K=K)
        close(got[t:t + 1], want)


def test_minimaxm3_indexer(ops):
    g = ops.gpu
    T, G, pos0, local, K = 3, 2, 3000, 2, 8
    n = pos0 + T
    nblk = (n + 127) // 128 + 1                         # one block wholly past the rows
    iq = orc.randn(44, (T, G, 128)); ik, _ = orc.randn_f16(45, (n, 128))
    bs = DevBuf(g, T * G * nblk * 4)
    ops.minimaxm3_idx_scores(DevBuf.of(g, iq), DevBuf.of(g, ik), bs, T, G, nblk, pos0, local)
    got = bs.read(np.float32).reshape(T, G, nblk)
    want = orc.mm3_idx_scores(iq, ik, T, G, nblk, pos0, local)
    fin = np.isfinite(want) & (want < 1e29)
    assert np.array_equal(np.isneginf(got), np.isneginf(want)) and np.array_equal(got > 1e29, want > 1e29)
    assert np.abs(got[fin] - want[fin]).max() < 1e-4
    # selection on the GPU's own scores against the oracle's selection on the same scores: bit for bit
    sel = DevBuf(g, T * G * K * 4)
    ops.minimaxm3_idx_topk(bs, sel, T, G, nblk, K)
    want_sel, want_left = orc.mm3_idx_topk(got, K)
    assert np.array_equal(sel.read(np.int32).reshape(T, G, K), want_sel)
    assert np.array_equal(bs.read(np.float32).reshape(T, G, nblk).view(np.uint32), want_left.view(np.uint32))
    # ties and exhaustion
    sc = np.array([[[1.0, 7.0, 7.0, -np.inf, 3.0, 7.0]]], np.float32)
    b2, s2 = DevBuf.of(g, sc), DevBuf(g, 6 * 4)
    ops.minimaxm3_idx_topk(b2, s2, 1, 1, 6, 6)
    assert s2.read(np.int32).tolist() == [1, 2, 5, 4, 0, -1]


@pytest.mark.parametrize("nblk,K", [(5, 8), (512, 16), (513, 16), (2048, 40), (2049, 3), (8192, 16), (8193, 5), (70, 70)])
def test_minimaxm3_topk_row_lengths(ops, nblk, K):
    """Every row length the selection has a kernel for (scores in 8, 32 or 128 registers a lane, or left in memory),
    on scores with ties, holes and boosted blocks: the lists and the scores left behind, bit for bit."""
    g = ops.gpu
    T, G = 2, 3
    rng = np.random.default_rng(nblk * 31 + K)
    sc = rng.integers(-50, 50, (T, G, nblk)).astype(np.float32) / 4            # many equal scores
    sc[rng.random((T, G, nblk)) < 0.2] = -np.inf
    sc[0, 0, : min(3, nblk)] += 1e30
    sc[1, 2] = -np.inf                                                         # a row with nothing to choose
    bs, sel = DevBuf.of(g, sc), DevBuf(g, T * G * K * 4)
    ops.minimaxm3_idx_topk(bs, sel, T, G, nblk, K)
    want_sel, want_left = orc.mm3_idx_topk(sc, K)
    assert np.array_equal(sel.read(np.int32).reshape(T, G, K), want_sel)
    assert np.array_equal(bs.read(np.float32).reshape(T, G, nblk).view(np.uint32), want_left.view(np.uint32))


@pytest.mark.parametrize("q8", [False, True])
@pytest.mark.parametrize("T,H,pos0,K", [(1, 128, 5000, 64), (3, 64, 2500, 512), (2, 160, 900, 16)])
def test_glm_cell_pools(ops, q8, T, H, pos0, K):
    g = ops.gpu
    L, scale = 512, 0.044
    n = pos0 + T
    qa = orc.randn(46, (T, H * L), 0.3)
    x = orc.randn(47, (n, L))
    if q8:
        rows = orc.glm_to_q8row(x, L)
    else:
        rows = orc.f2h(x).view(np.uint8).reshape(n, 2 * L)
    rng = np.random.default_rng(7)
    npool = (pos0 + 1) // 4
    sel = np.stack([rng.permutation(npool)[:K] if K <= npool else np.r_[rng.permutation(npool), [0] * (K - npool)] for _ in range(T)]).astype(np.int32)
    cnt = np.array([min(K, npool)] + [K // 3, -1][:T - 1], np.int32)          # a full list, a short one, a dense row
    u = DevBuf(g, T * H * L * 4); u.fill(0xFF)
    ops.mla_attend(DevBuf.of(g, qa), DevBuf.of(g, rows), u, T, H, L, pos0, scale, q8=q8, sel=DevBuf.of(g, sel), sel_cnt=DevBuf.of(g, cnt), K=K)
    want = orc.glm_mla_attend_sel(qa, rows, q8, T, H, L, pos0, scale, sel, cnt, K)
    close(u.read(np.float32).reshape(T, H * L), want)
    # no counts: the dense pass, as before
    ops.mla_attend(DevBuf.of(g, qa), DevBuf.of(g, rows), u, T, H, L, pos0, scale, q8=q8)
    close(u.read(np.float32).reshape(T, H * L), orc.glm_mla_attend(qa, rows, q8, T, H, L, pos0, scale).reshape(T, H * L))


def test_glm_dense_row_past_the_selection_bound_is_marked(ops):
    """A selection pass is sized for its lists and for dense rows of up to 2,560 cells (the reference's bound: its kernel
    keeps a row's scores in that many floats). A longer dense row must not come out as a plausible answer: NaNs."""
    g = ops.gpu
    T, H, L, pos0, K = 2, 16, 512, 2999, 16
    n = pos0 + T
    qa = orc.randn(1, (T, H * L), 0.3)
    rows = orc.f2h(orc.randn(2, (n, L))).view(np.uint8).reshape(n, 2 * L)
    sel = np.tile(np.arange(K, dtype=np.int32), (T, 1))
    cnt = np.array([K, -1], np.int32)                     # row 0 listed, row 1 dense over 3001 cells
    u = DevBuf(g, T * H * L * 4); u.fill(0)
    ops.mla_attend(DevBuf.of(g, qa), DevBuf.of(g, rows), u, T, H, L, pos0, 0.05, sel=DevBuf.of(g, sel), sel_cnt=DevBuf.of(g, cnt), K=K)
    got = u.read(np.float32).reshape(T, H * L)
    want = orc.glm_mla_attend_sel(qa, rows, False, T, H, L, pos0, 0.05, sel, cnt, K)
    close(got[:1], want.reshape(T, H * L)[:1])
    assert np.isnan(got[1]).all()


def test_glm_indexer_pools(ops):
    """ns_idx_pool over the engine's sequence of passes (a prompt chunk, then decode and verify passes whose pools reach
    back into the ring): pooled keys within float32 rounding of the oracle's (the exponential comes from another library),
    the ring byte for byte."""
    g = ops.gpu
    D, n_tok = 128, 213
    ik, ig, ape = orc.randn(5, (n_tok, D)), orc.randn(6, (n_tok, D)), orc.randn(7, (4, D), 0.5)
    ring = np.zeros((8, 2 * D), np.float32)
    pooled = np.zeros((n_tok // 4 + 1, D), np.float32)
    rb, pb, ab = DevBuf.of(g, ring), DevBuf.of(g, pooled), DevBuf.of(g, ape)
    pos = 0
    for T in (150, 1, 1, 3, 5, 1, 2, 4, 9, 16, 1, 20):
        orc.glm_idx_pool(ring, ik[pos:pos + T], ig[pos:pos + T], ape, pooled, pos, T, D)
        kb, gb = DevBuf.of(g, ik[pos:pos + T]), DevBuf.of(g, ig[pos:pos + T])
        ops.ok(ops.k.idx_pool(ops.raw(), rb.ptr, kb.ptr, gb.ptr, ab.ptr, pb.ptr, pos, T, D), "ns_idx_pool")
        pos += T
        assert np.array_equal(rb.read(np.float32).reshape(ring.shape), ring)
    assert pos == n_tok
    got = pb.read(np.float32).reshape(pooled.shape)
    assert np.abs(got - pooled).max() <= 4e-6 * np.abs(pooled).max()
    assert (got[n_tok // 4] == 0).all()


@pytest.mark.parametrize("T,H,j0,n,ld,pos0", [(1, 32, 0, 2500, 2500, 9999), (5, 32, 128, 300, 700, 1700), (40, 8, 0, 64, 80, 100)])
def test_glm_indexer_scores(ops, T, H, j0, n, ld, pos0):
    g = ops.gpu
    S, w = orc.randn(9, (T * H, n)), orc.randn(10, (T, H))
    score = np.full((T, ld), 3.0, np.float32)
    sb = DevBuf.of(g, score)
    orc.glm_idx_score(S, w, score, T, H, j0, n, pos0)
    Sb, wb = DevBuf.of(g, S), DevBuf.of(g, w)
    ops.ok(ops.k.idx_score(ops.raw(), Sb.ptr, wb.ptr, sb.ptr, T, H, j0, n, ld, pos0), "ns_idx_score")
    got = sb.read(np.float32).reshape(score.shape)
    fin = np.isfinite(score)
    assert np.array_equal(np.isneginf(got), np.isneginf(score))
    # (a head's product may be fused into the sum on one side and not on the other)
    assert np.abs(got[fin] - score[fin]).max() <= 1e-5 * max(1.0, float(np.abs(score[fin]).max()))
    with pytest.raises(Error, match="a pool range inside a score row"):
        ops.ok(ops.k.idx_score(ops.raw(), Sb.ptr, wb.ptr, sb.ptr, T, H, j0, n, j0 + n - 1, pos0), "ns_idx_score")


@pytest.mark.parametrize("T,n,K", [(1, 1, 1), (3, 7, 3), (2, 300, 40), (4, 5000, 512), (1, 5000, 4999), (2, 37, 37), (2, 20, 50), (1, 33000, 2048),
                                   (8, 1024, 1024), (3, 1025, 1), (2, 8192, 100), (2, 8193, 2048), (1, 32768, 2048), (2, 32769, 700), (1, 65536, 2048), (1, 65537, 300)])
def test_glm_top_k(ops, T, n, K):
    """ns_topk: the oracle's list bit for bit - on rows with many equal scores (the ties at the K-th value go to the lowest
    positions), -inf tails, fewer scores than K (the list's rest is left as it was) - and the same list on a second run."""
    g = ops.gpu
    rng = np.random.default_rng(n + K)
    ld = n + 6
    sc = rng.choice((np.round(rng.standard_normal(max(n // 3, 2)), 1) + 0.05).astype(np.float32), size=(T, ld)).astype(np.float32)
    if T > 1:
        sc[1, n // 2:n] = -np.inf
    if T > 2:
        sc[2, :n] = rng.standard_normal(n).astype(np.float32)    # all different
    want = orc.glm_topk(sc, n, K)
    scb = DevBuf.of(g, sc)
    for _ in range(2):
        sb = DevBuf.of(g, np.full((T, K), -1, np.int32))
        ops.ok(ops.k.topk(ops.raw(), scb.ptr, sb.ptr, T, n, ld, K), "ns_topk")
        assert np.array_equal(sb.read(np.int32).reshape(T, K), want)


def test_glm_indexer_feeds_the_latent_attention(ops):
    """The engine's sequence for a layer (llm/glm5next/src/engine.rs:1965-2013): pooled keys pass by pass, then for a verify
    pass the pool scores (the iq . pooled^T product is the engine's GEMM: taken here in numpy), the top pools a row, the
    counts - and ns_mla_attend_sel over those lists. The lists are the oracle's select of the scores the GPU produced, bit
    for bit; the attention is the oracle's over the same lists."""
    g = ops.gpu
    D, hh, kp, H, L = 128, 4, 16, 16, 512
    n_tok, T = 301, 3
    pos0 = n_tok - T
    ik, ig, ape = orc.randn(21, (n_tok, D)), orc.randn(22, (n_tok, D)), orc.randn(23, (4, D), 0.5)
    rb, pb, ab = DevBuf(g, 8 * 2 * D * 4), DevBuf(g, (n_tok // 4 + 1) * D * 4), DevBuf.of(g, ape)
    rb.fill(0)
    pb.fill(0)
    pos = 0
    for t in (200, 60, 38, T):
        kb, gb = DevBuf.of(g, ik[pos:pos + t]), DevBuf.of(g, ig[pos:pos + t])
        ops.ok(ops.k.idx_pool(ops.raw(), rb.ptr, kb.ptr, gb.ptr, ab.ptr, pb.ptr, pos, t, D), "ns_idx_pool")
        pos += t
    n = (pos0 + T) // 4
    assert n > kp
    pooled = pb.read(np.float32).reshape(-1, D)[:n]
    iq, w = orc.randn(24, (T * hh, D)), orc.randn(25, (T, hh))
    S = (iq @ pooled.T).astype(np.float32)                                   # [T hh][n]
    Sb, wb, scb, selb = DevBuf.of(g, S), DevBuf.of(g, w), DevBuf(g, T * n * 4), DevBuf.of(g, np.full((T, kp), -1, np.int32))
    ops.ok(ops.k.idx_score(ops.raw(), Sb.ptr, wb.ptr, scb.ptr, T, hh, 0, n, n, pos0), "ns_idx_score")
    ops.ok(ops.k.topk(ops.raw(), scb.ptr, selb.ptr, T, n, n, kp), "ns_topk")
    score = scb.read(np.float32).reshape(T, n)
    sel = selb.read(np.int32).reshape(T, kp)
    assert np.array_equal(sel, orc.glm_topk(score, n, kp))
    for r in range(T):
        assert (sel[r] < (pos0 + r + 1) // 4).all() and (np.diff(sel[r]) > 0).all()      # pools the row sees, in position order
    cnt = np.array([kp if (pos0 + r + 1) // 4 > kp else -1 for r in range(T)], np.int32)
    qa = orc.randn(26, (T, H * L), 0.3)
    rows = orc.f2h(orc.randn(27, (n_tok, L))).view(np.uint8).reshape(n_tok, 2 * L)
    u = DevBuf(g, T * H * L * 4)
    u.fill(0xFF)
    ops.mla_attend(DevBuf.of(g, qa), DevBuf.of(g, rows), u, T, H, L, pos0, 0.044, sel=selb, sel_cnt=DevBuf.of(g, cnt), K=kp)
    close(u.read(np.float32).reshape(T, H * L), orc.glm_mla_attend_sel(qa, rows, False, T, H, L, pos0, 0.044, sel, cnt, kp))


@pytest.mark.gpu
def test_glm_prompt_path_pieces(ops):
    """ns_mla_cells bit for bit and ns_softmax_masked within float32 rounding of the oracle: lists with room to spare and
    cut short, rows without lists, and score rows of every kernel form (kept in registers, and re-read)."""
    g = ops.gpu
    T, K, pos0 = 7, 9, 1234
    rng = np.random.default_rng(5)
    sel = rng.integers(0, (pos0 + 1) // 4, (T, K)).astype(np.int32)
    cnt = np.array([9, 0, -1, 4, 1, -1, 9], np.int32)
    for NC, lists in ((64, True), (17, True), (1280, True), (1280, False), (300, False)):
        ib, nb = DevBuf(g, T * NC * 4), DevBuf(g, T * 4)
        ib.fill(0xFF)
        nb.fill(0xFF)
        ops.mla_cells(T, K if lists else 0, pos0, ib, nb, NC, DevBuf.of(g, sel) if lists else None, DevBuf.of(g, cnt) if lists else None)
        want_i, want_n = orc.glm_mla_cells(T, K if lists else 0, pos0, NC, sel if lists else None, cnt if lists else None)
        assert np.array_equal(nb.read(np.int32), want_n), (NC, lists)
        assert np.array_equal(ib.read(np.int32).reshape(T, NC), want_i), (NC, lists)
    for R, H, NC, counts in ((3, 4, 64, (64, 0, 13)), (2, 3, 1024, (1000, 1)), (2, 2, 2112, (2051, 2112)), (2, 2, 5000, (4999, 300)), (1, 5, 257, (200,)),
                             (2, 1, 9000, (8999, 5)), (1, 2, 20000, (19998,)), (1, 2, 32768, (32768,)), (1, 2, 40000, (39990,)), (1, 2, 5001, (4000,)),
                             (1, 1, 17001, (17001,))):
        S = orc.randn(R + NC, (R * H, NC), 3.0)
        n = np.array(counts, np.int32)
        sb = DevBuf.of(g, S)
        ops.softmax_masked(sb, R, H, NC, DevBuf.of(g, n), 0.29)
        got = sb.read(np.float32).reshape(R * H, NC)
        want = orc.glm_softmax_masked(S, R, H, NC, n, 0.29)
        assert np.array_equal(got == 0.0, want == 0.0) or np.abs(got - want).max() < 1e-7
        # (the oracle, as the reference's work-item does, adds a row's exponentials one after another in float32: over
        # thousands of cells its own sum drifts, so long rows are also held to the float64 closed form of the same
        # float32 scaled scores)
        assert np.abs(got - want).max() <= 2e-6 * max(1.0, (NC / 1024.0) ** 0.5) * max(want.max(), 1e-30) + 1e-9, (R, H, NC)
        x = (S * np.float32(0.29)).astype(np.float64)
        for rh in range(R * H):
            m = n[rh // H]
            if m:
                e = np.exp(x[rh, :m] - x[rh, :m].max())
                assert np.abs(got[rh, :m] - e / e.sum()).max() <= 2e-6 * (e / e.sum()).max() + 1e-12, (R, H, NC, rh)
        for rh in range(R * H):
            assert not got[rh, n[rh // H]:].any()
            if n[rh // H]:
                assert abs(got[rh].sum() - 1.0) < 1e-5
