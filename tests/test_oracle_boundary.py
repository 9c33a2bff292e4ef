"""Pins the oracle's restatements behind the entry points added for the boundary row - the draft block with one first
key (ns_mm3s_attend_block), ns_q35_attn_probs, ns_mla_attend, ns_gather_q8_h - against numpy float64 straight from their
definitions and hand-derived known answers. No GPU."""
import numpy as np

from oracle import orc


def _softmax_rows(s):
    e = np.exp(s - s.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


def test_block_closed_form_against_the_definition():
    T, Hq, Hkv, D, p0, w0 = 5, 4, 2, 128, 300, 37
    cap = p0 + T
    k, v = orc.randn(1, (cap, Hkv * D)), orc.randn(2, (cap, Hkv * D))
    kc, vc = orc.kv_store(0, k, v, Hkv, D, cap, 0)
    q = orc.randn(3, (T, Hq * D))
    kf = orc.h2f(kc.view(np.uint16)).reshape(Hkv, cap, D).astype(np.float64)
    vf = orc.h2f(vc.view(np.uint16)).reshape(Hkv, cap, D).astype(np.float64)
    want = np.zeros((T, Hq, D))
    for h in range(Hq):
        hk = h // (Hq // Hkv)
        s = q.reshape(T, Hq, D)[:, h].astype(np.float64) @ kf[hk, w0:cap].T / np.sqrt(D)
        want[:, h] = _softmax_rows(s) @ vf[hk, w0:cap]
    got = orc.attn_f64_block(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0, w0)
    assert np.abs(got.reshape(T, Hq, D) - want).max() < 1e-12
    # first key 0 = the plain pass that is not causal; a wrong first key (one off) must show
    assert np.array_equal(orc.attn_f64_block(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0, 0), orc.attn_f64(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0, causal=False))
    assert np.abs(orc.attn_f64_block(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0, w0 + 1).reshape(T, Hq, D) - want).max() > 1e-6


def test_attn_probs_against_the_definition():
    Hq, Hkv, D, cap, n = 6, 2, 256, 700, 613
    for kt in (0, 1, 2):
        k = orc.randn(10 + kt, (cap, Hkv * D))
        kc, _ = orc.kv_store(kt, k, k, Hkv, D, cap, 0)
        q = orc.randn(20 + kt, (Hq, D), 0.5)
        kf = orc.kv_dequant(kc.reshape(Hkv * cap, -1), kt, D).reshape(Hkv, cap, D).astype(np.float64)
        p = np.stack([_softmax_rows(q[h].astype(np.float64) @ kf[h // (Hq // Hkv), :n].T / np.sqrt(D)) for h in range(Hq)])
        base = np.linspace(0.0, 1.0, n).astype(np.float32)
        for mode, want in ((0, p.mean(0)), (1, p.max(0))):
            got = orc.attn_probs(kt, q, kc, Hq, Hkv, D, cap, n, mode, out=base)
            assert np.abs(got - (base + want)).max() < 2e-6, (kt, mode)
        # the mean of softmax rows sums to one over the keys
        assert abs(orc.attn_probs(kt, q, kc, Hq, Hkv, D, cap, n, 0).sum() - 1.0) < 1e-4
    # one key: every head gives it weight 1 whatever the mode
    one = orc.attn_probs(0, orc.randn(5, (Hq, D)), orc.kv_store(0, k[:1], k[:1], Hkv, D, 1, 0)[0], Hq, Hkv, D, 1, 1, 1)
    assert one.tolist() == [1.0]


def test_glm_dense_f32_cache_against_the_definition():
    T, H, L, pos0, scale = 3, 5, 512, 200, 0.05
    n = pos0 + T
    qa, c = orc.randn(31, (T, H, L), 0.4), orc.randn(32, (n, L))
    got = orc.glm_mla_attend_f32(qa, c, T, H, L, pos0, scale)
    for t in range(T):
        s = qa[t].astype(np.float64) @ c[: pos0 + t + 1].astype(np.float64).T * scale
        want = _softmax_rows(s) @ c[: pos0 + t + 1].astype(np.float64)
        assert np.abs(got[t] - want).max() < 5e-6


def test_gather_q8_known_answers():
    L = 512
    row = np.zeros((3, 32 + L), np.uint8)
    sc = row[:, :32].view(np.uint16)
    sc[0, :] = orc.f2h(np.array([0.5], np.float32))[0]
    sc[1, :] = orc.f2h(np.array([0.0123], np.float32))[0]
    sc[2, 3] = orc.f2h(np.array([2.0], np.float32))[0]
    row[0, 32:] = np.arange(L, dtype=np.int64).astype(np.uint8)          # q = 0 .. 127, -128 .. -1, ...
    row[1, 32:] = 127
    row[2, 32 + 96: 32 + 128] = np.uint8(0x81)                            # -127 in block 3
    out = orc.glm_gather_q8_h(row, np.array([2, 0, 1, 0], np.int32), L)
    f = orc.h2f(out)
    assert f.shape == (4, L)
    assert np.array_equal(f[1], 0.5 * np.arange(L).astype(np.uint8).view(np.int8).astype(np.float32)) and np.array_equal(f[1], f[3])
    assert np.array_equal(f[0, 96:128], np.full(32, -254.0, np.float32)) and not f[0, :96].any() and not f[0, 128:].any()
    d = orc.h2f(sc[1, :1])[0]
    assert np.array_equal(out[2], np.full(L, np.float16(np.float32(d) * np.float32(127)).view(np.uint16)))
    # against numpy's own rounding for a random row made by the (pinned) quantizer
    y = orc.glm_to_q8row(orc.randn(7, (5, L)), L)
    want = (orc.h2f(y[:, :32].view(np.uint16).copy()).repeat(32, axis=1) * y[:, 32:].view(np.int8).astype(np.float32)).astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.glm_gather_q8_h(y, np.arange(5, dtype=np.int32), L), want)


def _q6k_numpy(blocks):
    """ggml dequantize_row_q6_K restated in numpy. blocks uint8 [nb][210] -> float32 [nb][256]:
    for each half n (128 values) and l = 0..31: q1 = (ql[l] & 15) | ((qh[l] >> 0) & 3) << 4, q2 = (ql[l + 32] & 15) | ((qh[l] >> 2) & 3) << 4,
    q3 = (ql[l] >> 4) | ((qh[l] >> 4) & 3) << 4, q4 = (ql[l + 32] >> 4) | ((qh[l] >> 6) & 3) << 4, each less 32;
    y[l + 32 g] = d * sc[l / 16 + 2 g] * q_g."""
    nb = blocks.shape[0]
    ql = blocks[:, :128].astype(np.int32).reshape(nb, 2, 64)
    qh = blocks[:, 128:192].astype(np.int32).reshape(nb, 2, 32)
    sc = blocks[:, 192:208].view(np.int8).astype(np.float32).reshape(nb, 2, 8)
    d = blocks[:, 208:210].copy().view(np.float16).astype(np.float32).reshape(nb, 1, 1)
    out = np.zeros((nb, 2, 4, 32), np.float32)
    is_ = np.arange(32) // 16
    for g, (src, hi, sh) in enumerate(((ql[:, :, :32], False, 0), (ql[:, :, 32:], False, 2), (ql[:, :, :32], True, 4), (ql[:, :, 32:], True, 6))):
        lo = (src >> 4) if hi else (src & 15)
        q = (lo | (((qh >> sh) & 3) << 4)) - 32
        out[:, :, g, :] = (d * sc[:, :, is_ + 2 * g]).astype(np.float32) * q.astype(np.float32)
    return out.reshape(nb, 256)


def random_q6k_rows(seed, n):
    """n Q6_K rows of 512 values: random 6-bit values and scales, d near 1e-3 (the size of real kv_b weights)."""
    rng = np.random.default_rng(seed)
    b = np.zeros((n * 2, 210), np.uint8)
    b[:, :192] = rng.integers(0, 256, (n * 2, 192), dtype=np.uint8)
    b[:, 192:208] = rng.integers(-60, 61, (n * 2, 16)).astype(np.int8).view(np.uint8)
    b[:, 208:210] = (rng.uniform(5e-4, 2e-3, n * 2).astype(np.float16)).view(np.uint8).reshape(n * 2, 2)
    return b.reshape(n, 420)


def test_q6k_rows_against_the_published_rule():
    rows = random_q6k_rows(5, 40)
    rows[0].reshape(2, 210)[:, :192] = 0
    rows[1].reshape(2, 210)[:, :192] = 0xFF
    want = _q6k_numpy(rows.reshape(-1, 210)).reshape(40, 512)
    assert np.array_equal(orc.q6k_rows512(rows), want)
    # all-zero ql / qh: every value is -32 times its block's d x scale
    ds = np.repeat(rows[0].reshape(2, 210)[:, 192:208].view(np.int8).astype(np.float32), 16, axis=1) * rows[0].reshape(2, 210)[:, 208:210].copy().view(np.float16).astype(np.float32)
    assert np.array_equal(want[0].reshape(2, 256), ds * np.float32(-32.0))
    assert np.array_equal(want[1].reshape(2, 256), np.repeat(rows[1].reshape(2, 210)[:, 192:208].view(np.int8).astype(np.float32), 16, axis=1) *
                          rows[1].reshape(2, 210)[:, 208:210].copy().view(np.float16).astype(np.float32) * np.float32(31.0))


def test_q6k_absorb_and_value_projection_against_the_definition():
    T, H = 2, 3
    kvb = random_q6k_rows(6, H * 256).reshape(H, 256, 420)
    q = orc.randn(7, (T, H, 192))
    w = orc.q6k_rows512(kvb).reshape(H, 256, 512).astype(np.float64)
    qa = orc.mla_absorb_q6k(q, kvb, T, H)
    want = np.einsum("hic,thi->thc", w[:, :128], q[:, :, :128].astype(np.float64))
    assert np.abs(qa[:, :, :512] - want).max() < 1e-4 * np.abs(want).max() and np.array_equal(qa[:, :, 512:], q[:, :, 128:])
    u = orc.randn(8, (T, H, 512))
    out = orc.mla_vb_q6k(u, kvb, T, H)
    want = np.einsum("hvc,thc->thv", w[:, 128:], u.astype(np.float64))
    assert np.abs(out - want).max() < 1e-4 * np.abs(want).max()
