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
    assert seen == 2


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
