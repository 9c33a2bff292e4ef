"""Pins the oracle's sparse-selection restatements (MiniMax-M3 block lists + indexer, GLM cell pools) without the
reference: against the dense forms already pinned, against float64 closed forms over the selected keys written in numpy,
and by the selection's own invariants (order of the list, holes, ties)."""
import numpy as np

from oracle import orc


def closed_form(q, k, v, scale):
    """softmax(q k^T scale) v in float64: q [D], k / v [n][D]."""
    s = (k.astype(np.float64) @ q.astype(np.float64)) * scale
    w = np.exp(s - s.max())
    return (w[:, None] * v.astype(np.float64)).sum(0) / w.sum()


def test_mm3_block_lists():
    T, H, G, pos0, scale = 2, 8, 2, 700, 0.09
    n = pos0 + T
    q = orc.randn(1, (T, H * 128))
    kc, kf = orc.randn_f16(2, (n, G, 128)); vc, vf = orc.randn_f16(3, (n, G, 128))
    nblk = (n + 127) // 128
    dense = orc.mm3_attend(q, kc, vc, T, H, G, pos0, scale)
    # every block, in order: the dense result (the same keys in the same chunks)
    allb = np.tile(np.arange(nblk, dtype=np.int32), (T, G, 1))
    assert np.allclose(orc.mm3_attend(q, kc, vc, T, H, G, pos0, scale, sel=allb, K=nblk), dense, atol=1e-6)
    # any order, holes (-1) anywhere: float32 reassociation only
    perm = allb[:, :, ::-1].copy()
    holes = np.concatenate([perm[:, :, :2], np.full((T, G, 3), -1, np.int32), perm[:, :, 2:]], -1)
    assert np.allclose(orc.mm3_attend(q, kc, vc, T, H, G, pos0, scale, sel=holes, K=nblk + 3), dense, atol=2e-6)
    # a true subset against the closed form over exactly its keys (the last block is cut at the row's position)
    sel = np.array([[[5, 0, -1], [2, 5, 1]], [[5, 3, 4], [-1, -1, 0]]], np.int32)
    got = orc.mm3_attend(q, kc, vc, T, H, G, pos0, scale, sel=sel, K=3).reshape(T, H, 128)
    for t in range(T):
        for h in range(H):
            gi = h // (H // G)
            keys = np.concatenate([np.arange(b * 128, min((b + 1) * 128, pos0 + t + 1)) for b in sel[t, gi] if b >= 0])
            want = closed_form(q[t, h * 128:(h + 1) * 128], kf[keys, gi], vf[keys, gi], scale)
            assert np.abs(got[t, h] - want).max() < 2e-5
    # nothing selected: zeros
    none = np.full((T, G, 2), -1, np.int32)
    assert not orc.mm3_attend(q, kc, vc, T, H, G, pos0, scale, sel=none, K=2).any()


def test_mm3_indexer():
    T, G, pos0, local = 3, 2, 1000, 2
    n = pos0 + T
    nblk = (n + 127) // 128
    iq = orc.randn(4, (T, G, 128)); ik, ikf = orc.randn_f16(5, (n, 128))
    bs = orc.mm3_idx_scores(iq, ik, T, G, nblk, pos0, local)
    dots = np.einsum("tgd,jd->tgj", iq.astype(np.float64), ikf.astype(np.float64))
    for t in range(T):
        pos = pos0 + t
        for b in range(nblk):
            want = dots[t, :, b * 128:min((b + 1) * 128, pos + 1)].max(-1)
            if b + local > pos // 128:
                assert (bs[t, :, b] > 9e29).all() and np.allclose(bs[t, :, b] - np.float32(1e30), 0, atol=1e24)   # the bonus swallows the score
            else:
                assert np.abs(bs[t, :, b] - want).max() < 1e-4
    # a block wholly past the row
    assert np.isneginf(orc.mm3_idx_scores(iq, ik, T, G, nblk + 2, pos0, local)[:, :, nblk:]).all()
    # top-k: best first, the lowest index of equal scores, -1 when nothing finite is left; picked scores become -inf
    sc = np.array([[[1.0, 7.0, 7.0, -np.inf, 3.0, 7.0]]], np.float32)
    sel, left = orc.mm3_idx_topk(sc, 6)
    assert sel.tolist() == [[[1, 2, 5, 4, 0, -1]]] and np.isneginf(left).all()
    sel, _ = orc.mm3_idx_topk(bs, 4)
    order = np.argsort(-bs, axis=-1, kind="stable")[:, :, :4]
    assert np.array_equal(sel, order)


def test_glm_cell_pools():
    T, H, L, pos0, scale = 3, 4, 512, 97, 0.05
    n = pos0 + T
    qa = orc.randn(6, (T, H * L), 0.3); cache, cf = orc.randn_f16(7, (n, L))
    raw = cache.view(np.uint8)
    dense = orc.glm_mla_attend(qa, raw, False, T, H, L, pos0, scale).reshape(T, H * L)
    K = 40
    # every complete pool, in order + the row's incomplete pool = every cell, in order: the dense result exactly
    cnt = np.array([(pos0 + t + 1) // 4 for t in range(T)], np.int32)
    sel = np.tile(np.arange(K, dtype=np.int32), (T, 1))
    assert np.array_equal(orc.glm_mla_attend_sel(qa, raw, False, T, H, L, pos0, scale, sel, cnt, K), dense)
    # a negative count: dense
    assert np.array_equal(orc.glm_mla_attend_sel(qa, raw, False, T, H, L, pos0, scale, sel, np.full(T, -1, np.int32), K), dense)
    # a few pools against the closed form over exactly their cells
    sel = np.array([[3, 20, 7] + [0] * (K - 3)] * T, np.int32); cnt = np.array([3, 2, 0], np.int32)
    got = orc.glm_mla_attend_sel(qa, raw, False, T, H, L, pos0, scale, sel, cnt, K).reshape(T, H, L)
    for t in range(T):
        p = pos0 + t
        cells = [4 * int(b) + i for b in sel[t, :cnt[t]] for i in range(4)] + list(range(4 * ((p + 1) // 4), p + 1))
        for h in range(H):
            if cells:
                want = closed_form(qa[t, h * L:(h + 1) * L], cf[cells], cf[cells], scale)
                assert np.abs(got[t, h] - want).max() < 2e-5
            else:
                assert not got[t, h].any()


def _glm_indexer_inputs(seed, n_tok, D):
    return orc.randn(seed, (n_tok, D)), orc.randn(seed + 1, (n_tok, D)), orc.randn(seed + 2, (4, D), 0.5)


def test_glm_indexer_pools_in_closed_form():
    """orc.glm_idx_pool (kernels/llm/glm5next/glm.cpp:883-916) against the softmax written out in float64, fed as the
    engine feeds it: a prompt chunk, then passes of 1, 3 and 5 tokens whose pools' earlier members come from the ring;
    the ring holds the last 8 tokens, ik | ig, at slot position % 8."""
    D, n_tok = 24, 61
    ik, ig, ape = _glm_indexer_inputs(5, n_tok, D)
    ring = np.zeros((8, 2 * D), np.float32)
    pooled = np.full((n_tok // 4 + 1, D), np.nan, np.float32)
    pos = 0
    for T in (18, 1, 3, 5, 1, 1, 1, 2, 4, 9, 16):
        orc.glm_idx_pool(ring, ik[pos:pos + T], ig[pos:pos + T], ape, pooled, pos, T, D)
        pos += T
        for p in range(max(0, pos - 8), pos):
            assert np.array_equal(ring[p % 8, :D], ik[p]) and np.array_equal(ring[p % 8, D:], ig[p])
    assert pos == n_tok
    for j in range(n_tok // 4):
        lg = ig[4 * j:4 * j + 4].astype(np.float64) + ape
        wgt = np.exp(lg - lg.max(axis=0))
        want = (wgt * ik[4 * j:4 * j + 4]).sum(axis=0) / wgt.sum(axis=0)
        assert np.abs(pooled[j] - want).max() < 1e-5, j
    assert np.isnan(pooled[n_tok // 4]).all()                # the incomplete pool is not written


def test_glm_indexer_scores_and_top_k():
    """orc.glm_idx_score: the relu-weighted head sum in float64, -inf for the pools a row does not see yet, columns
    outside [j0, j0 + n) untouched. orc.glm_topk: the K largest as ascending positions, ties at the K-th value to the
    lowest positions - against a stable sort, on rows with many equal scores, -inf tails and fewer scores than K."""
    T, H, j0, n, ld, pos0 = 5, 6, 3, 20, 40, 70
    S = orc.randn(9, (T * H, n))
    w = orc.randn(10, (T, H))
    score = np.full((T, ld), 7.0, np.float32)
    orc.glm_idx_score(S, w, score, T, H, j0, n, pos0)
    for r in range(T):
        nv = (pos0 + r + 1) // 4
        want = (np.maximum(S[r * H:(r + 1) * H].astype(np.float64), 0.0) * w[r].astype(np.float64)[:, None]).sum(axis=0)
        for jj in range(n):
            if j0 + jj < nv:
                assert abs(score[r, j0 + jj] - want[jj]) < 1e-5
            else:
                assert score[r, j0 + jj] == -np.inf
        assert (score[r, :j0] == 7.0).all() and (score[r, j0 + n:] == 7.0).all()
    rng = np.random.default_rng(3)
    for n, K in ((1, 1), (7, 3), (300, 40), (5000, 512), (5000, 4999), (37, 37), (20, 50)):
        sc = rng.choice(np.round(rng.standard_normal(max(n // 3, 2)), 1).astype(np.float32) + 0.05, size=(3, n + 5)).astype(np.float32)
        sc[1, n // 2:n] = -np.inf                            # the pools a row does not see yet
        sel = orc.glm_topk(sc, n, K)
        for r in range(3):
            order = np.lexsort((np.arange(n), -sc[r, :n].astype(np.float64)))      # by score descending, then position
            want = np.sort(order[:min(K, n)])
            assert np.array_equal(sel[r, :min(K, n)], want), (n, K, r)
            assert (sel[r, min(K, n):] == -1).all()


def _cells_of(pos, pools):
    """A row's cells from the statement of the selection: the 4 tokens of each listed pool, then the tokens of the row's
    incomplete pool; no list: every cell up to the row's own."""
    if pools is None:
        return list(range(pos + 1))
    return [4 * int(b) + i for b in pools for i in range(4)] + list(range(4 * ((pos + 1) // 4), pos + 1))


def test_glm_cells_and_masked_softmax():
    """ns_mla_cells / ns_softmax_masked (kernels/llm/glm5next/glm.cpp:1023-1060): the lists against the selection spelt out
    in Python, the softmax against scipy's in float64 - and the chain they belong to (gather, scores, softmax, weighted sum
    in numpy) against the latent attention over the same lists."""
    from scipy.special import softmax
    T, K, pos0 = 5, 6, 41
    sel = np.array([[9, 2, 5, 0, 1, 3], [1, 0, 7, 4, 9, 8], [3, 3, 3, 3, 3, 3], [0, 1, 2, 3, 4, 5], [8, 6, 4, 2, 0, 1]], np.int32)
    cnt = np.array([3, 6, 0, -1, 2], np.int32)
    for NC in (64, 16, 1):                                                   # room for every cell; lists cut short
        idx, n = orc.glm_mla_cells(T, K, pos0, NC, sel, cnt)
        for t in range(T):
            cells = _cells_of(pos0 + t, None if cnt[t] < 0 else sel[t, :cnt[t]])
            assert n[t] == min(len(cells), NC)
            assert idx[t].tolist() == (cells + [0] * NC)[:NC]
    idx, n = orc.glm_mla_cells(T, 0, pos0, 64)                                # no lists at all: dense rows
    for t in range(T):
        assert n[t] == pos0 + t + 1 and idx[t, :n[t]].tolist() == list(range(pos0 + t + 1)) and not idx[t, n[t]:].any()

    R, H, NC, scale = 4, 3, 40, 0.37
    S = orc.randn(3, (R * H, NC), 4.0)
    S[1] += 300.0                                                            # large scores: the maximum is taken off first
    m = np.array([40, 17, 0, 1], np.int32)
    got = orc.glm_softmax_masked(S, R, H, NC, m, scale)
    for rh in range(R * H):
        k = m[rh // H]
        assert not got[rh, k:].any()
        if k:
            assert np.abs(got[rh, :k] - softmax(S[rh, :k].astype(np.float64) * scale)).max() < 2e-6

    # the chain of the prompt path: cells -> gathered latents -> scores -> masked softmax -> weighted latents
    T, Hh, L, K, pos0, scale = 3, 2, 512, 4, 30, 0.05
    ncell = pos0 + T
    qa = orc.randn(6, (T, Hh * L), 0.3)
    cache, cf = orc.randn_f16(7, (ncell, L))
    sel = np.array([[5, 1, 3, 0], [2, 6, 0, 1], [0, 0, 0, 0]], np.int32)
    cnt = np.array([4, 2, -1], np.int32)
    NC = 64
    idx, n = orc.glm_mla_cells(T, K, pos0, NC, sel, cnt)
    sc = np.stack([qa[t].reshape(Hh, L) @ cf[idx[t]].T for t in range(T)]).astype(np.float32)      # [T][Hh][NC]
    pr = orc.glm_softmax_masked(sc.reshape(T * Hh, NC), T, Hh, NC, n, scale).reshape(T, Hh, NC)
    u = np.stack([pr[t] @ cf[idx[t]] for t in range(T)]).reshape(T, Hh * L)
    want = orc.glm_mla_attend_sel(qa, cache.view(np.uint8), False, T, Hh, L, pos0, scale, sel, cnt, K)
    assert np.abs(u - want).max() < 2e-5
