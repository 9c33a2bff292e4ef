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
