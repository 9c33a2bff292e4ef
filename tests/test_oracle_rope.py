"""Pins the oracle's norm + rotary-position restatements (oracle/oracle.c: orc_q35_norm_rope, orc_mg_norm_rope,
orc_mm3_norm_rope_row) without the reference: a float64 complex-rotation statement written straight from the definition,
and the rotation's invariants - chosen so that a wrong sign, a wrong pairing, a wrong exponent or a dropped weight fails."""
import numpy as np
import pytest

from oracle import orc


def rms(x, w, eps):
    x = x.astype(np.float64)
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * w.astype(np.float64)


def rot_half(v, n_rot, ang):
    """v [..., D]; pairs (i, i + n_rot / 2) of the first n_rot turned by ang [..., n_rot / 2] (float64)."""
    hr = n_rot // 2
    z = (v[..., :hr] + 1j * v[..., hr:n_rot]) * np.exp(1j * ang)
    out = v.copy()
    out[..., :hr], out[..., hr:n_rot] = z.real, z.imag
    return out


@pytest.mark.parametrize("D,n_rot", [(64, 64), (128, 64), (256, 64), (128, 128), (128, 0)])
def test_q35_norm_rope_against_the_definition(D, n_rot):
    T, H, p0, theta, eps = 5, 3, 7, 10000.0, 1e-6
    x = orc.randn(1, (T, H, D)); w = 1.0 + 0.1 * orc.randn(2, (D,))
    got = orc.q35_norm_rope(x, T, H, D, w, eps, n_rot, theta, p0).reshape(T, H, D)
    v = rms(x, w, eps)
    if n_rot:
        k = np.arange(n_rot // 2)
        ang = (p0 + np.arange(T))[:, None, None] * theta ** (-2.0 * k / n_rot)[None, None, :]
        v = rot_half(v, n_rot, ang)
    assert np.abs(got - v).max() < 2e-5                      # float32 angles at positions <= 11
    # without the norm (ns_q35_rope)
    got2 = orc.q35_norm_rope(x, T, H, D, None, eps, n_rot, theta, p0).reshape(T, H, D)
    v2 = x.astype(np.float64)
    if n_rot:
        v2 = rot_half(v2, n_rot, ang)
    assert np.abs(got2 - v2).max() < 2e-5


def test_rotation_invariants():
    T, H, D, n_rot, theta = 4, 2, 128, 64, 1e6
    x = orc.randn(3, (T, H, D)); w = np.ones(D, np.float32)
    # position 0 turns nothing: the result is the RMS norm exactly (cos 0 = 1, sin 0 = 0)
    y0 = orc.q35_norm_rope(x[:1], 1, H, D, w, 1e-6, n_rot, theta, 0).reshape(1, H, D)
    assert np.abs(y0 - rms(x[:1], w, 1e-6)).max() < 1e-6
    # a pair's length is kept, features past n_rot are untouched
    y = orc.q35_norm_rope(x, T, H, D, None, 0.0, n_rot, theta, 1000).reshape(T, H, D)
    hr = n_rot // 2
    assert np.allclose(y[..., :hr] ** 2 + y[..., hr:n_rot] ** 2, x[..., :hr] ** 2 + x[..., hr:n_rot] ** 2, rtol=1e-5)
    assert np.array_equal(y[..., n_rot:], x[..., n_rot:])
    # the dot product of two rotated rows depends on the distance only (what makes it a position encoding)
    a = orc.q35_norm_rope(x[:1], 1, H, D, None, 0.0, n_rot, theta, 5).reshape(H, D)
    b = orc.q35_norm_rope(x[1:2], 1, H, D, None, 0.0, n_rot, theta, 9).reshape(H, D)
    a2 = orc.q35_norm_rope(x[:1], 1, H, D, None, 0.0, n_rot, theta, 105).reshape(H, D)
    b2 = orc.q35_norm_rope(x[1:2], 1, H, D, None, 0.0, n_rot, theta, 109).reshape(H, D)
    assert np.allclose((a * b).sum(-1), (a2 * b2).sum(-1), atol=2e-4)


def test_q35_positions_with_sections():
    # text rows (all three positions equal) come out as the plain form at that position; with distinct positions pair k
    # turns by the one its section names: sections (2, 1, 1) -> k % 4 = 0 -> t, 1 -> h, 2 -> w, 3 -> t
    T, H, D, n_rot, theta = 3, 2, 128, 64, 10000.0
    x = orc.randn(4, (T, H, D)); w = 1.0 + 0.1 * orc.randn(5, (D,))
    pos = np.array([[5, 5, 5], [6, 6, 6], [7, 7, 7]], np.int32)
    a = orc.q35_norm_rope(x, T, H, D, w, 1e-6, n_rot, theta, 0, pos3=pos, sections=(2, 1, 1))
    b = orc.q35_norm_rope(x, T, H, D, w, 1e-6, n_rot, theta, 5)
    assert np.array_equal(a, b)
    pos = np.array([[3, 11, 20], [4, 12, 21], [5, 13, 22]], np.int32)
    got = orc.q35_norm_rope(x, T, H, D, w, 1e-6, n_rot, theta, 0, pos3=pos, sections=(2, 1, 1)).reshape(T, H, D)
    k = np.arange(n_rot // 2)
    which = np.array([0, 1, 2, 0])[k % 4]
    ang = pos[:, which][:, None, :] * theta ** (-2.0 * k / n_rot)[None, None, :]
    assert np.abs(got - rot_half(rms(x, w, 1e-6), n_rot, ang)).max() < 5e-5


@pytest.mark.parametrize("rope", [0, 1, 2])
def test_mg_norm_rope_against_the_definition(rope):
    T, H, D, theta, p0, eps = 4, 3, 128, 10000.0, 3, 1e-5
    x = orc.randn(6, (T, H, D)); w = 1.0 + 0.1 * orc.randn(7, (D,))
    got = orc.mg_norm_rope(x, T, H, D, w, eps, rope, theta, p0).reshape(T, H, D)
    v = rms(x, w, eps)
    i = np.arange(D // 2)
    ang = (p0 + np.arange(T))[:, None, None] * theta ** (-2.0 * i / D)[None, None, :]
    if rope == 1:        # adjacent pairs
        z = (v[..., 0::2] + 1j * v[..., 1::2]) * np.exp(1j * ang)
        v = np.stack([z.real, z.imag], -1).reshape(T, H, D)
    elif rope == 2:      # halves
        v = rot_half(v, D, ang)
    assert np.abs(got - v).max() < 2e-5


def test_mm3_rows():
    HD, n_rot, base, eps, pos = 128, 64, 5e6, 1e-6, 9
    x = orc.randn(8, (HD,)); w = 1.0 + 0.1 * orc.randn(9, (HD,))
    k = np.arange(n_rot // 2)
    ang = pos * base ** (-2.0 * k / n_rot)
    # plain in-place rotation (ns_llm_minimaxm3_rope)
    y, _ = orc.mm3_norm_rope_row(x, None, True, n_rot, pos, base, eps)
    assert np.abs(y - rot_half(x.astype(np.float64), n_rot, ang)).max() < 2e-5
    # norm + rotation + half copy (ns_mm3s_attn_post's q / k rows)
    y, h = orc.mm3_norm_rope_row(x, w, True, n_rot, pos, base, eps, want_half=True)
    assert np.abs(y - rot_half(rms(x, w, eps), n_rot, ang)).max() < 2e-5
    assert np.array_equal(h, orc.f2h(y))
    # a value row: untouched, stored as half
    y, h = orc.mm3_norm_rope_row(x, None, False, n_rot, pos, base, eps, want_half=True)
    assert np.array_equal(y, x) and np.array_equal(h, orc.f2h(x))
