"""The step in front of attention (q / k RMS norm, rotary positions, KV store) on the GPU against the oracle, and the
fused launch against the separate calls bit for bit.

Tolerance of the float32 stage: the angle pos * theta^(-2k/n) is a float32 product whose factors come from powf, cosf
and sinf implementations that differ between the CPU's libm and the GPU's by an ulp; an ulp of the angle is
pos * 2^-23 radians, so the bound is 4 (1 + pos) 2^-23 max|v| + 2e-6 max|v| (written below as `tol`)."""
import numpy as np
import pytest

from nextsycl_amd import DevBuf
from nextsycl_amd.attn import kv_row_bytes
from oracle import orc

pytestmark = pytest.mark.gpu


def tol(ref, pos):
    return (4.0 * (1.0 + pos) * 2.0 ** -23 + 2e-6) * np.abs(ref).max()


@pytest.mark.parametrize("D,n_rot,p0", [(128, 64, 3), (256, 64, 4095), (128, 128, 100000), (64, 32, 17), (128, 0, 5),
                                        # rotated widths that are not whole 4-feature groups (the feature-by-feature
                                        # instance), and heads past 256 features (two groups a lane), both ways
                                        (128, 20, 9), (64, 6, 1000), (512, 64, 77), (384, 20, 5), (48, 12, 30)])
def test_q35_norm_rope(ops, D, n_rot, p0):
    g = ops.gpu
    T, H, theta, eps = 6, 5, 1e6, 1e-6
    # the engine's q comes out of a fused [q | gate] projection: heads 2 D apart in src
    src = orc.randn(11, (T, H, 2 * D)); w = (1.0 + 0.1 * orc.randn(12, (D,))).astype(np.float32)
    x = np.ascontiguousarray(src[:, :, :D])
    dst = DevBuf(g, T * H * D * 4); dst.fill(0xFF)
    ops.q35_qk_norm_rope(DevBuf.of(g, src), H * 2 * D, 2 * D, dst, H * D, T, H, D, DevBuf.of(g, w), eps, n_rot, theta, p0)
    want = orc.q35_norm_rope(x, T, H, D, w, eps, n_rot, theta, p0)
    got = dst.read(np.float32).reshape(T, H * D)
    assert np.abs(got - want).max() <= tol(want, p0 + T)
    # the plain rotation
    ops.q35_qk_norm_rope(DevBuf.of(g, x), H * D, D, dst, H * D, T, H, D, None, 0.0, n_rot, theta, p0)
    want = orc.q35_norm_rope(x, T, H, D, None, 0.0, n_rot, theta, p0)
    assert np.abs(dst.read(np.float32).reshape(T, H * D) - want).max() <= tol(want, p0 + T)


def test_q35_positions(ops):
    g = ops.gpu
    T, H, D, n_rot, theta, eps = 4, 3, 128, 64, 1e6, 1e-6
    x = orc.randn(13, (T, H * D)); w = (1.0 + 0.1 * orc.randn(14, (D,))).astype(np.float32)
    pos = np.array([[3, 11, 20], [4, 12, 21], [5, 5, 5], [900, 7, 64]], np.int32)
    dst = DevBuf(g, T * H * D * 4)
    ops.q35_qk_norm_rope(DevBuf.of(g, x), H * D, D, dst, H * D, T, H, D, DevBuf.of(g, w), eps, n_rot, theta, 0, pos3=DevBuf.of(g, pos), sections=(2, 1, 1))
    want = orc.q35_norm_rope(x, T, H, D, w, eps, n_rot, theta, 0, pos3=pos, sections=(2, 1, 1))
    assert np.abs(dst.read(np.float32).reshape(T, H * D) - want).max() <= tol(want, 900)


@pytest.mark.parametrize("rope", [0, 1, 2])
def test_mg_norm_rope_in_place(ops, rope):
    g = ops.gpu
    T, H, D, theta, eps, p0 = 5, 16, 128, 10000.0, 1e-5, 777
    x = orc.randn(15, (T, H * D)); w = (1.0 + 0.1 * orc.randn(16, (D,))).astype(np.float32)
    xb = DevBuf.of(g, x)
    ops.mg_qk_norm_rope(xb, H * D, xb, H * D, T, H, D, DevBuf.of(g, w), eps, rope, theta, p0)     # y = x, as the engine calls it
    want = orc.mg_norm_rope(x, T, H, D, w, eps, rope, theta, p0)
    assert np.abs(xb.read(np.float32).reshape(T, H * D) - want).max() <= tol(want, p0 + T)


@pytest.mark.parametrize("n_rot", [64, 20])        # whole 4-feature groups, and a width that is not
def test_minimaxm3_rope_and_attn_post(ops, n_rot):
    g = ops.gpu
    H, G, IH, HD, base, eps, pos = 8, 2, 3, 128, 5e6, 1e-6, 4321
    T, row = 3, H * HD + 64
    x = orc.randn(17, (T, row))
    xb = DevBuf.of(g, x)
    ops.minimaxm3_rope(xb, T, H, row, HD, n_rot, 100, base)
    got = xb.read(np.float32).reshape(T, row)
    for t in range(T):
        for h in range(H):
            want, _ = orc.mm3_norm_rope_row(x[t, h * HD:(h + 1) * HD], None, True, n_rot, 100 + t, base, eps)
            assert np.abs(got[t, h * HD:(h + 1) * HD] - want).max() <= tol(want, 100 + t)
        assert np.array_equal(got[t, H * HD:], x[t, H * HD:])                    # past the heads: untouched
    # the decode token's fused step
    q, k, v = orc.randn(18, (H, HD)), orc.randn(19, (G, HD)), orc.randn(20, (G, HD))
    iq, ik = orc.randn(21, (IH, HD)), orc.randn(22, (HD,))
    ws = [(1.0 + 0.1 * orc.randn(23 + i, (HD,))).astype(np.float32) for i in range(4)]
    cap = 8
    kc, vc, ic = DevBuf(g, cap * G * HD * 2), DevBuf(g, cap * G * HD * 2), DevBuf(g, cap * HD * 2)
    for b in (kc, vc, ic):
        b.fill(0xEE)
    slot = 5
    qb, kb, vb, iqb, ikb = (DevBuf.of(g, a) for a in (q, k, v, iq, ik))
    ops.mm3s_attn_post(qb, kb, vb, iqb, ikb, *(DevBuf.of(g, w) for w in ws), (kc, slot * G * HD * 2), (vc, slot * G * HD * 2), (ic, slot * HD * 2),
                       H, G, IH, HD, n_rot, pos, base, eps)
    t = lambda ref: tol(ref, pos)
    gq, gk, gv = qb.read(np.float32).reshape(H, HD), kb.read(np.float32).reshape(G, HD), vb.read(np.float32).reshape(G, HD)
    giq, gik = iqb.read(np.float32).reshape(IH, HD), ikb.read(np.float32)
    hk = kc.read(np.uint16).reshape(cap, G, HD); hv = vc.read(np.uint16).reshape(cap, G, HD); hi = ic.read(np.uint16).reshape(cap, HD)
    for h in range(H):
        want, _ = orc.mm3_norm_rope_row(q[h], ws[0], True, n_rot, pos, base, eps)
        assert np.abs(gq[h] - want).max() <= t(want)
    for j in range(G):
        want, _ = orc.mm3_norm_rope_row(k[j], ws[1], True, n_rot, pos, base, eps)
        assert np.abs(gk[j] - want).max() <= t(want)
        assert np.array_equal(hk[slot, j], orc.f2h(gk[j]))                      # the half row is the float32 row, rounded
        assert np.array_equal(hv[slot, j], orc.f2h(v[j])) and np.array_equal(gv[j], v[j])
    for h in range(IH):
        want, _ = orc.mm3_norm_rope_row(iq[h], ws[2], True, n_rot, pos, base, eps)
        assert np.abs(giq[h] - want).max() <= t(want)
    want, _ = orc.mm3_norm_rope_row(ik, ws[3], True, n_rot, pos, base, eps)
    assert np.abs(gik - want).max() <= t(want) and np.array_equal(hi[slot], orc.f2h(gik))
    assert (hk[:slot] == 0xEEEE).all() and (hk[slot + 1:] == 0xEEEE).all() and (hi[:slot] == 0xEEEE).all()   # other rows untouched


@pytest.mark.parametrize("kt", [0, 1, 2, 3])
@pytest.mark.parametrize("rope,D,n_rot", [(1, 128, 64), (1, 256, 64), (2, 128, 0), (3, 128, 0), (1, 64, 64)])
def test_fused_equals_the_separate_calls_bit_for_bit(ops, kt, rope, D, n_rot):
    g = ops.gpu
    T, Hq, Hkv, cap, p0, theta, eps = 7, 8, 2, 64, 50, 1e6, 1e-6
    ring = rope != 1 and kt in (0, 3)            # the separate store keeps rings for 16-bit rows only
    if ring:
        p0 = 60                                                                  # wraps: slots 60..63, 0..2
    q, k, v = orc.randn(31, (T, Hq * D)), orc.randn(32, (T, Hkv * D)), orc.randn(33, (T, Hkv * D))
    qw, kw = ((1.0 + 0.1 * orc.randn(34 + i, (D,))).astype(np.float32) for i in range(2))
    qb, kb, vb, qwb, kwb = (DevBuf.of(g, a) for a in (q, k, v, qw, kw))
    # ---- separate: two norm + rope launches into float32, then the store
    qo, kn = DevBuf(g, T * Hq * D * 4), DevBuf(g, T * Hkv * D * 4)
    if rope == 1:
        ops.q35_qk_norm_rope(qb, Hq * D, D, qo, Hq * D, T, Hq, D, qwb, eps, n_rot, theta, p0)
        ops.q35_qk_norm_rope(kb, Hkv * D, D, kn, Hkv * D, T, Hkv, D, kwb, eps, n_rot, theta, p0)
    else:
        ops.mg_qk_norm_rope(qb, Hq * D, qo, Hq * D, T, Hq, D, qwb, eps, rope - 1, theta, p0)
        ops.mg_qk_norm_rope(kb, Hkv * D, kn, Hkv * D, T, Hkv, D, kwb, eps, rope - 1, theta, p0)
    nb = Hkv * cap * kv_row_bytes(kt, D)
    kc1, vc1, kc2, vc2 = (DevBuf(g, nb) for _ in range(4))
    for b in (kc1, vc1, kc2, vc2):
        b.fill(0xC3)
    ops.kv_store(kt, kn, Hkv * D, vb, Hkv * D, T, Hkv, D, cap, p0, kc1, vc1, ring=ring)
    # ---- fused
    qo2 = DevBuf(g, T * Hq * D * 4)
    ops.pre_store(rope, 0, kt, ring, qb, Hq * D, D, qo2, Hq * D, kb, Hkv * D, D, vb, Hkv * D, qwb, kwb, eps, n_rot, theta, T, Hq, Hkv, D, cap, p0, kc2, vc2)
    assert np.array_equal(qo.read(np.uint32), qo2.read(np.uint32))
    assert np.array_equal(kc1.read(np.uint8), kc2.read(np.uint8))
    assert np.array_equal(vc1.read(np.uint8), vc2.read(np.uint8))
    # and 16-bit query rows are the float32 rows, rounded
    for qt, conv in ((1, orc.f2h), (2, orc.f2bf)):
        qo3 = DevBuf(g, T * Hq * D * 2)
        ops.pre_store(rope, qt, kt, ring, qb, Hq * D, D, qo3, Hq * D, kb, Hkv * D, D, vb, Hkv * D, qwb, kwb, eps, n_rot, theta, T, Hq, Hkv, D, cap, p0, kc2, vc2)
        assert np.array_equal(qo3.read(np.uint16), conv(qo.read(np.float32)))


@pytest.mark.parametrize("kt", [0, 1, 2, 3])
@pytest.mark.parametrize("rope,D,n_rot", [(1, 64, 32), (1, 128, 64), (3, 128, 0), (1, 256, 64)])
def test_a_prompt_pass_equals_its_rows_in_small_passes(ops, kt, rope, D, n_rot):
    """A prompt-sized pass has each wave walk several heads of its rows (across the q / k / v groups) and, for heads of
    64 and 128, several rows at once; a pass of 100 rows takes a wave a head. Both must give the same bytes. The row
    count leaves the last wave's row group part empty."""
    g = ops.gpu
    T, Hq, Hkv, p0, theta, eps, step = 3001, 6, 3, 11, 1e6, 1e-6, 100
    cap = p0 + T
    q, k, v = orc.randn(41, (T, Hq * D)), orc.randn(42, (T, Hkv * D)), orc.randn(43, (T, Hkv * D))
    qw, kw = ((1.0 + 0.1 * orc.randn(44 + i, (D,))).astype(np.float32) for i in range(2))
    qb, kb, vb, qwb, kwb = (DevBuf.of(g, a) for a in (q, k, v, qw, kw))
    nb = Hkv * cap * kv_row_bytes(kt, D)
    kc1, vc1, kc2, vc2 = (DevBuf(g, nb) for _ in range(4))
    for b in (kc1, vc1, kc2, vc2):
        b.fill(0x5A)
    qo1, qo2 = DevBuf(g, T * Hq * D * 2), DevBuf(g, T * Hq * D * 2)
    ops.pre_store(rope, 1, kt, False, qb, Hq * D, D, qo1, Hq * D, kb, Hkv * D, D, vb, Hkv * D, qwb, kwb, eps, n_rot, theta, T, Hq, Hkv, D, cap, p0, kc1, vc1)
    for t0 in range(0, T, step):
        n = min(step, T - t0)
        ops.pre_store(rope, 1, kt, False, qb.view(t0 * Hq * D * 4, n * Hq * D * 4), Hq * D, D, qo2.view(t0 * Hq * D * 2, n * Hq * D * 2), Hq * D,
                      kb.view(t0 * Hkv * D * 4, n * Hkv * D * 4), Hkv * D, D, vb.view(t0 * Hkv * D * 4, n * Hkv * D * 4), Hkv * D, qwb, kwb, eps, n_rot,
                      theta, n, Hq, Hkv, D, cap, p0 + t0, kc2, vc2)
    assert np.array_equal(qo1.read(np.uint16), qo2.read(np.uint16))
    assert np.array_equal(kc1.read(np.uint8), kc2.read(np.uint8))
    assert np.array_equal(vc1.read(np.uint8), vc2.read(np.uint8))
    # and the rows are the oracle's: the last ones, where the angle is largest
    if rope == 1 and kt == 0:
        lo = T - 4
        want = orc.q35_norm_rope(q[lo:], 4, Hq, D, qw, eps, n_rot, theta, p0 + lo)
        got = orc.h2f(qo1.read(np.uint16).reshape(T, Hq * D)[lo:])
        assert np.abs(got - want).max() <= tol(want, p0 + T) + 2.0 ** -11 * np.abs(want).max()


def test_pre_store_at_bench_size(ops):
    """bench.py's `pre_store8k` at its full size (8192 rows, 40 q / 8 kv heads of 128, bfloat16 rows and cache): the
    caches bit for bit what the separate calls store, q rows bit for bit the separate call's float32 rows rounded, and
    sampled rows against the oracle."""
    g = ops.gpu
    T, Hq, Hkv, D, n_rot, theta, eps, p0, kt = 8192, 40, 8, 128, 64, 1e6, 1e-6, 0, 3
    cap = T
    q, k, v = orc.randn(51, (T, Hq * D)), orc.randn(52, (T, Hkv * D)), orc.randn(53, (T, Hkv * D))
    qw, kw = ((1.0 + 0.1 * orc.randn(54 + i, (D,))).astype(np.float32) for i in range(2))
    qb, kb, vb, qwb, kwb = (DevBuf.of(g, a) for a in (q, k, v, qw, kw))
    nb = Hkv * cap * kv_row_bytes(kt, D)
    kc1, vc1, kc2, vc2 = (DevBuf(g, nb) for _ in range(4))
    qo = DevBuf(g, T * Hq * D * 2)
    ops.pre_store(1, 2, kt, False, qb, Hq * D, D, qo, Hq * D, kb, Hkv * D, D, vb, Hkv * D, qwb, kwb, eps, n_rot, theta, T, Hq, Hkv, D, cap, p0, kc1, vc1)
    qf, kn = DevBuf(g, T * Hq * D * 4), DevBuf(g, T * Hkv * D * 4)
    ops.q35_qk_norm_rope(qb, Hq * D, D, qf, Hq * D, T, Hq, D, qwb, eps, n_rot, theta, p0)
    ops.q35_qk_norm_rope(kb, Hkv * D, D, kn, Hkv * D, T, Hkv, D, kwb, eps, n_rot, theta, p0)
    ops.kv_store(kt, kn, Hkv * D, vb, Hkv * D, T, Hkv, D, cap, p0, kc2, vc2)
    assert np.array_equal(kc1.read(np.uint8), kc2.read(np.uint8))
    assert np.array_equal(vc1.read(np.uint8), vc2.read(np.uint8))
    got = qo.read(np.uint16).reshape(T, Hq * D)
    assert np.array_equal(got, orc.f2bf(qf.read(np.float32)).reshape(T, Hq * D))
    for t in (0, 1, 4097, T - 1):
        want = orc.q35_norm_rope(q[t:t + 1], 1, Hq, D, qw, eps, n_rot, theta, p0 + t)
        assert np.abs(orc.bf2f(got[t:t + 1]) - want).max() <= tol(want, p0 + t) + 2.0 ** -8 * np.abs(want).max()


def test_pre_store_rejects_bad_arguments(ops):
    from nextsycl_amd import Error
    g = ops.gpu
    b = DevBuf(g, 1 << 16)
    with pytest.raises(Error):
        ops.pre_store(1, 0, 0, False, b, 128, 128, b, 128, b, 128, 128, b, 128, b, b, 1e-6, 64, 1e4, 1, 1, 1, 96, 16, 0, b, b)    # D = 96
    with pytest.raises(Error):
        ops.pre_store(1, 0, 0, False, b, 128, 128, b, 128, b, 128, 128, b, 128, b, b, 1e-6, 64, 1e4, 4, 1, 1, 128, 16, 14, b, b)  # past capacity
    with pytest.raises(Error):
        ops.pre_store(1, 0, 0, False, b, 128, 128, b, 128, b, 128, 128, b, 128, b, b, 1e-6, 63, 1e4, 1, 1, 1, 128, 16, 0, b, b)   # odd n_rot
