"""The oracle against the committed golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the
definitions in numpy): cache bytes bit for bit, the float64 closed forms to 1e-12, the reference-order float32 kernels to
reassociation error. The fixtures' own checksums are checked first, so neither side can drift unnoticed."""
import hashlib
import os

import numpy as np
import pytest

from oracle import orc

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = ["decode", "verify", "window", "prompt", "wide"]


def load(name):
    return np.load(os.path.join(GOLD, name), allow_pickle=False)


def test_manifest():
    lines = open(os.path.join(GOLD, "MANIFEST.sha256")).read().split("\n")
    seen = 0
    for ln in lines:
        if not ln.strip():
            continue
        digest, fn = ln.split()
        assert hashlib.sha256(open(os.path.join(GOLD, fn), "rb").read()).hexdigest() == digest, fn
        seen += 1
    assert seen == 3


@pytest.mark.parametrize("kt", [0, 1, 2, 3])
@pytest.mark.parametrize("case", CASES)
def test_cache_bytes_and_attention(case, kt):
    z = load("attention.npz")
    T, Hq, Hkv, D, p0, win = (int(x) for x in z[case + "_shape"])
    cap = p0 + T
    kc, vc = orc.kv_store(kt, z[case + "_k"], z[case + "_v"], Hkv, D, cap, 0)
    assert np.array_equal(kc, z["%s_kc%d" % (case, kt)]) and np.array_equal(vc, z["%s_vc%d" % (case, kt)])
    q = z[case + "_q"] if kt != 3 else orc.bf2f(orc.f2bf(z[case + "_q"]))
    want = z["%s_out%d" % (case, kt)]
    assert np.abs(orc.attn_f64(q, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win) - want).max() < 1e-12
    mx, rel, _ = orc.compare(orc.attn_exact(q, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=win), want)
    assert mx < 5e-6 and rel < 5e-6


def test_mla_and_glm_rows():
    z = load("mla.npz")
    T, H, pos0 = (int(x) for x in z["shape"])
    scale = float(z["scale"][0])
    u64 = orc.mla_f64(z["qa"], z["cache"], T, H, pos0, scale, 512, 64)
    assert np.abs(u64 - z["u"]).max() < 1e-12
    assert orc.compare(orc.mla_decode_u(z["qa"], z["cache"], T, H, pos0, scale), z["u"])[0] < 5e-6
    assert np.array_equal(orc.glm_to_q8row(z["glm_x"], 512), z["glm_rows"])


def test_rope_and_indexer():
    z = load("select.npz")
    T, H, head, off, n_dims, pos0 = (int(x) for x in z["rope_shape"])
    y = orc.ds2_rope(z["rope_x"].copy(), T, H, H * head, head, off, n_dims, pos0, *(float(v) for v in z["rope_yarn"]))
    assert np.abs(y - z["rope_y"]).max() < 1e-4 * np.abs(z["rope_x"]).max() * float(z["rope_yarn"][3])     # float32 angles near 1000 radians
    D, n_tok, hh, K, Tq, q0 = (int(x) for x in z["idx_shape"])
    ring = np.zeros((8, 2 * D), np.float32)
    pooled = np.zeros((n_tok // 4, D), np.float32)
    pos = 0
    for t in (30, 1, 2, 5, 12):
        orc.glm_idx_pool(ring, z["idx_ik"][pos:pos + t], z["idx_ig"][pos:pos + t], z["idx_ape"], pooled, pos, t, D)
        pos += t
    assert pos == n_tok and np.abs(pooled - z["idx_pooled"]).max() < 1e-5
    npool = n_tok // 4
    score = np.zeros((Tq, npool), np.float32)
    orc.glm_idx_score(z["idx_S"], z["idx_w"], score, Tq, hh, 0, npool, q0)
    want = z["idx_score"]
    assert np.array_equal(np.isneginf(score), np.isneginf(want))
    assert np.abs(score[np.isfinite(want)] - want[np.isfinite(want)]).max() < 1e-5
    assert np.array_equal(orc.glm_topk(z["idx_score32"], npool, K), z["idx_sel"])
