"""Pins the oracle's attention functions: the float64 closed form against an independent numpy evaluation, the
reference-order float32 restatements against it, invariants (weights sum to one, partition invariance of the split
merge, window and ring handling, empty visibility), MLA against its closed form."""
import numpy as np
import pytest

from oracle import orc


def _numpy_attention(q, K, V, Hq, Hkv, D, p0, win=0, causal=True, scale=None, T=None):
    """softmax(q K^T s + mask) V in float64, straight from the definition. K, V: [Hkv][positions][D] float."""
    T = q.shape[0]
    G = Hq // Hkv
    s = scale if scale else 1.0 / np.sqrt(D)
    out = np.zeros((T, Hq, D))
    for r in range(T):
        pos = p0 + r
        end = pos + 1 if causal else p0 + T
        first = max(0, pos + 1 - win) if win > 0 else 0
        for h in range(Hq):
            k, v = K[h // G, first:end].astype(np.float64), V[h // G, first:end].astype(np.float64)
            if len(k) == 0:
                continue
            sc = k @ q[r, h * D:(h + 1) * D].astype(np.float64) * s
            e = np.exp(sc - sc.max())
            out[r, h] = (e / e.sum()) @ v
    return out.reshape(T, Hq * D)


@pytest.mark.parametrize("kt", [0, 1, 2, 3])
@pytest.mark.parametrize("T,Hq,Hkv,D,p0,win", [(1, 8, 2, 128, 300, 0), (5, 6, 3, 64, 40, 0), (3, 4, 1, 128, 500, 128), (4, 12, 2, 256, 77, 0)])
def test_closed_form_and_exact_restatement(kt, T, Hq, Hkv, D, p0, win):
    cap = p0 + T
    k, v = orc.randn(1, (cap, Hkv * D)), orc.randn(2, (cap, Hkv * D))
    q = orc.randn(3, (T, Hq * D))
    kc, vc = orc.kv_store(kt, k, v, Hkv, D, cap, 0)
    K, V = orc.kv_dequant(kc, kt, D), orc.kv_dequant(vc, kt, D)
    want = _numpy_attention(q, K, V, Hq, Hkv, D, p0, win)
    f64 = orc.attn_f64(q, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
    assert np.abs(f64 - want).max() < 1e-12
    ex = orc.attn_exact(q, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win)
    mx, rel, cos = orc.compare(ex, want)
    assert mx < 5e-6 and rel < 5e-6                       # float32 in another order: reassociation only
    if D % 2 == 0:
        fl = orc.attn_flash_model(q, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win, kbs=64)
        mx, rel, cos = orc.compare(fl, want)
        assert mx < 2e-3 and rel < (1e-3 if kt != 3 else 1e-3 + 2.0 ** -9)    # the XMX kernels' 16-bit operand model


def test_weights_sum_to_one_and_empty_rows():
    T, Hq, Hkv, D, p0 = 3, 4, 2, 128, 100
    cap = p0 + T
    k = orc.randn(1, (cap, Hkv * D))
    v = np.ones((cap, Hkv * D), np.float32)
    kc, vc = orc.kv_store(0, k, v, Hkv, D, cap, 0)
    q = orc.randn(3, (T, Hq * D), 3.0)
    assert np.abs(orc.attn_f64(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0) - 1).max() < 1e-12
    assert np.abs(orc.attn_exact(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0) - 1).max() < 1e-6
    assert np.abs(orc.attn_flash_model(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0, kbs=64) - 1).max() < 5e-4   # P is rounded to half, l is not
    # T = 0: nothing computed, nothing written
    assert orc.attn_exact(np.zeros((0, Hq * D), np.float32), kc, vc, 0, 0, Hq, Hkv, D, cap, 0).size == 0


def test_split_merge_is_partition_invariant():
    """Any cut of the keys into splits merges to the unsplit result (to float32 rounding): exact kernel with the
    reference's decode splits against one split, flash model with several split sizes."""
    T, Hq, Hkv, D, p0 = 1, 8, 2, 128, 3000
    cap = p0 + T
    k, v = orc.randn(1, (cap, Hkv * D)), orc.randn(2, (cap, Hkv * D))
    q = orc.randn(3, (T, Hq * D))
    kc, vc = orc.kv_store(0, k, v, Hkv, D, cap, 0)
    ref = orc.attn_f64(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0)
    a = orc.attn_exact(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0, groups=2)        # many splits of 32
    b = orc.attn_exact(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0, groups=2, split_single_only=True)
    c = orc.attn_exact(np.repeat(q, 2, 0), kc, vc, 0, 2, Hq, Hkv, D, cap, p0 - 1, groups=2, split_single_only=True)   # T = 2: unsplit (q35 rule)
    for x in (a, b):
        assert orc.compare(x, ref)[0] < 5e-6
    assert orc.compare(c[1:], ref)[0] < 5e-6
    outs = [orc.attn_flash_model(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0, kbs=kbs) for kbs in (0, 64, 128, 1024)]
    for o in outs[1:]:
        assert np.abs(o - outs[0]).max() < 1e-4      # the weights are rounded to half against another running maximum


def test_ring_slots_and_position_major():
    T, Hq, Hkv, D, cap, win, p0 = 2, 4, 2, 128, 64, 50, 150
    k, v = orc.randn(1, (p0 + T, Hkv * D)), orc.randn(2, (p0 + T, Hkv * D))
    kc = np.zeros((Hkv, cap, 2 * D), np.uint8)
    vc = np.zeros((Hkv, cap, 2 * D), np.uint8)
    for s in range(0, p0 + T, 16):
        e = min(p0 + T, s + 16)
        orc.kv_store(0, k[s:e], v[s:e], Hkv, D, cap, s, kc, vc, ring=True)
    q = orc.randn(3, (T, Hq * D))
    got = orc.attn_f64(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0, win=win)
    K = orc.h2f(orc.f2h(k)).reshape(-1, Hkv, D).transpose(1, 0, 2)
    V = orc.h2f(orc.f2h(v)).reshape(-1, Hkv, D).transpose(1, 0, 2)
    assert np.abs(got - _numpy_attention(q, K, V, Hq, Hkv, D, p0, win)).max() < 1e-12
    # position-major [pos][Hkv][D] gives the same as head-major
    cap2 = p0 + T
    kc2, vc2 = orc.kv_store(0, k, v, Hkv, D, cap2, 0)
    a = orc.attn_f64(q, kc2, vc2, 0, T, Hq, Hkv, D, cap2, p0, scale=0.05)
    b = orc.attn_f64(q, np.ascontiguousarray(kc2.transpose(1, 0, 2)), np.ascontiguousarray(vc2.transpose(1, 0, 2)), 0, T, Hq, Hkv, D, cap2, p0, pm=True, scale=0.05)
    assert np.array_equal(a, b)
    m = orc.mm3_attend(q, np.ascontiguousarray(kc2.transpose(1, 0, 2)).view(np.uint16), np.ascontiguousarray(vc2.transpose(1, 0, 2)).view(np.uint16), T, Hq, Hkv, p0, 0.05)
    assert orc.compare(m, a)[0] < 5e-6
    with pytest.raises(ValueError):
        orc.kv_store(0, k, v, Hkv, D, 10, 0)              # past the capacity


def test_not_causal_block():
    T, Hq, Hkv, D, p0 = 4, 4, 1, 128, 60
    cap = p0 + T
    k, v = orc.randn(1, (cap, Hkv * D)), orc.randn(2, (cap, Hkv * D))
    q = orc.randn(3, (T, Hq * D))
    kc, vc = orc.kv_store(0, k, v, Hkv, D, cap, 0)
    K, V = orc.kv_dequant(kc, 0, D), orc.kv_dequant(vc, 0, D)
    want = _numpy_attention(q, K, V, Hq, Hkv, D, p0, causal=False)
    assert np.abs(orc.attn_f64(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0, causal=False) - want).max() < 1e-12
    assert orc.compare(orc.attn_exact(q, kc, vc, 0, T, Hq, Hkv, D, cap, p0, causal=False), want)[0] < 5e-6


# ---- MLA -----------------------------------------------------------------------------------------------------------------------
def test_mla_decode_against_closed_form():
    T, H, L, R, NOPE, V, pos0 = 2, 6, 512, 64, 128, 128, 70
    n = pos0 + T
    cache = orc.f2h(orc.randn(1, (n, L + R), 0.5))
    q = orc.randn(2, (T, H, NOPE + R))
    kb = orc.f2h(orc.randn(3, (H, L, NOPE), 0.1))
    vb = orc.f2h(orc.randn(4, (H, V, L), 0.1))
    scale = 1.0 / np.sqrt(192.0)
    qa = orc.mla_absorb(q, kb, T, H, L, R, NOPE)
    # the absorb is a plain mat-vec
    want_qa = np.einsum("hrc,thc->thr", orc.h2f(kb).astype(np.float64), q[:, :, :NOPE].astype(np.float64))
    assert np.abs(qa[:, :, :L] - want_qa).max() < 1e-4 and np.array_equal(qa[:, :, L:], q[:, :, NOPE:])
    u = orc.mla_decode_u(qa, cache, T, H, pos0, scale, L, R)
    u64 = orc.mla_f64(qa, cache, T, H, pos0, scale, L, R)
    c = orc.h2f(cache).astype(np.float64)
    for t in range(T):
        for h in range(H):
            s = c[:pos0 + t + 1] @ qa[t, h].astype(np.float64) * scale
            e = np.exp(s - s.max())
            assert np.abs(u64[t, h] - (e / e.sum()) @ c[:pos0 + t + 1, :L]).max() < 1e-12
    assert orc.compare(u, u64)[0] < 5e-6
    out = orc.mla_vb(u, vb, T, H, L, V)
    want = np.einsum("hvl,thl->thv", orc.h2f(vb).astype(np.float64), u.astype(np.float64))
    assert np.abs(out - want).max() < 1e-4


def test_glm_latent_mla_and_q8_rows():
    T, H, L, pos0 = 2, 4, 512, 90
    n = pos0 + T
    x = orc.randn(1, (n, L), 0.5)
    qa = orc.randn(2, (T, H, L))
    half = orc.f2h(x)
    u = orc.glm_mla_attend(qa, half, False, T, H, L, pos0, 0.04)
    u64 = orc.mla_f64(qa, half, T, H, pos0, 0.04, L, 0)
    assert orc.compare(u, u64)[0] < 5e-6
    rows = orc.glm_to_q8row(x, L)
    deq = np.repeat(rows[:, :32].view(np.float16).astype(np.float32), 32, axis=1) * rows[:, 32:].view(np.int8).astype(np.float32)
    u8 = orc.glm_mla_attend(qa, rows, True, T, H, L, pos0, 0.04)
    want = orc.mla_f64(qa, orc.f2h(deq), T, H, pos0, 0.04, L, 0)     # the dequantized values need not be halves: tolerance
    assert orc.compare(u8, want)[0] < 2e-3
    assert np.abs(deq - x).max() <= np.abs(x).max() / 127 * 0.51 + 1e-3


def test_ds2_kv_store_reduces_to_textbook_rope():
    """ext_factor 0, freq_scale 1, mscale 1: RMS norm x weight on the latent, plain RoPE on adjacent pairs of the key."""
    T, L, R, pos0 = 3, 512, 64, 17
    kv = orc.randn(1, (T, L + R))
    w = orc.randn(2, (L,), 0.3) + 1.0
    cache = np.zeros((pos0 + T, L + R), np.uint16)
    orc.ds2_kv_store(kv, w, 1e-6, cache, T, L, R, pos0, 10000.0, 1.0, 0.0, 1.0, 0.0, 0.0)
    got = orc.h2f(cache[pos0:])
    x = kv.astype(np.float64)
    lat = x[:, :L] / np.sqrt((x[:, :L] ** 2).mean(axis=1, keepdims=True) + 1e-6) * w
    assert np.abs(got[:, :L] - lat).max() < 2e-3            # half rounding of values up to ~4
    i = np.arange(R // 2)
    for t in range(T):
        ang = (pos0 + t) * 10000.0 ** (-2.0 * i / R)
        x0, x1 = x[t, L::2], x[t, L + 1::2]
        assert np.abs(got[t, L::2] - (x0 * np.cos(ang) - x1 * np.sin(ang))).max() < 3e-3
        assert np.abs(got[t, L + 1::2] - (x0 * np.sin(ang) + x1 * np.cos(ang))).max() < 3e-3
    assert (cache[:pos0] == 0).all()


def test_ds2_rope_is_ggml_yarn_in_closed_form():
    """orc.ds2_rope (and with it the angle code ds2_kv_store shares) against ggml's rope_yarn written out in float64: the
    extrapolated angle pos * base^(-i0 / n), the interpolated one freq_scale times it, their mix by the ramp between the
    correction dims times ext_factor, cos and sin times mscale - with the mix switched on, off, and a plain rope; the
    rotated slice only, the copy to `out`, every other float untouched."""
    T, H, row, head, off, n, pos0 = 5, 3, 3 * 40 + 7, 40, 8, 24, 4000
    for base, fs, ext, ms, c0, c1 in ((10000.0, 1.0, 0.0, 1.0, 0.0, 0.0), (10000.0, 0.025, 1.0, 1.3, 3.0, 9.0), (5.0e5, 0.5, 0.4, 0.8, 2.0, 6.5)):
        x = orc.randn(3, (T, row))
        out = np.full((T, H, n), 7.0, np.float32)
        got = orc.ds2_rope(x.copy(), T, H, row, head, off, n, pos0, base, fs, ext, ms, c0, c1, out, H * n, n)
        want = x.astype(np.float64)
        i = np.arange(n // 2)
        ramp = 1.0 - np.clip((i - c0) / max(0.001, c1 - c0), 0.0, 1.0)
        for t in range(T):
            extrap = (pos0 + t) * base ** (-2.0 * i / n)
            interp = fs * extrap
            theta = interp * (1 - ramp * ext) + extrap * ramp * ext if ext != 0.0 else interp
            c, s_ = np.cos(theta) * ms, np.sin(theta) * ms
            for h in range(H):
                a = x[t, h * head + off:h * head + off + n].astype(np.float64)
                want[t, h * head + off:h * head + off + n:2] = a[0::2] * c - a[1::2] * s_
                want[t, h * head + off + 1:h * head + off + n:2] = a[0::2] * s_ + a[1::2] * c
        # (float32 angles of a few thousand radians: 2^-12 radians an ulp, a few of them by the repeated products)
        assert np.abs(got - want).max() < 4e-4 * np.abs(x).max() * max(1.0, ms)
        rot = np.zeros((T, row), bool)
        for h in range(H):
            rot[:, h * head + off:h * head + off + n] = True
        assert np.array_equal(got[~rot], x[~rot])
        for h in range(H):
            assert np.array_equal(out[:, h], got[:, h * head + off:h * head + off + n])
    # small positions: the float32 chain is then tight against float64
    x = orc.randn(4, (2, 64))
    got = orc.ds2_rope(x.copy(), 2, 1, 64, 64, 0, 64, 3, 10000.0, 0.25, 1.0, 1.2, 10.0, 23.0)
    i = np.arange(32)
    ramp = 1.0 - np.clip((i - 10.0) / 13.0, 0.0, 1.0)
    for t in range(2):
        extrap = (3 + t) * 10000.0 ** (-2.0 * i / 64)
        theta = 0.25 * extrap * (1 - ramp) + extrap * ramp
        a = x[t].astype(np.float64)
        assert np.abs(got[t, 0::2] - (a[0::2] * np.cos(theta) - a[1::2] * np.sin(theta)) * 1.2).max() < 1e-5
        assert np.abs(got[t, 1::2] - (a[0::2] * np.sin(theta) + a[1::2] * np.cos(theta)) * 1.2).max() < 1e-5
