"""Shared by the parity tests: seeded inputs from the oracle's generator, caches packed by the oracle's stores, the
HIP path called through the C ABI wrappers, and the comparison measures (max-abs, relative L2) with the tolerances of
the path: max-abs 2e-3 and relative L2 1e-3 against the float64 closed form for float32 / half outputs."""
import numpy as np

from nextsycl_amd import DevBuf
from nextsycl_amd.attn import BF16, F16, F32, kv_row_bytes
from oracle import orc

MAX_ABS, REL_L2 = 2e-3, 1e-3
# a bfloat16 output adds its own rounding (8 bits of significand): half an ulp is 2^-9 relative
BF16_ROUND = 2.0 ** -9

SEED_Q, SEED_K, SEED_V = 0xA11CE, 0xB0B, 0xC0FFEE


def make_kv(kt, Hkv, D, cap, nkeys, cfg=0, sigma=1.0, pm=False):
    """Caches holding positions 0..nkeys-1, packed by the oracle: (kc, vc) uint8. Head-major [Hkv][cap][row] or
    position-major [cap][Hkv][row]."""
    k = orc.randn(SEED_K + cfg, (nkeys, Hkv * D), sigma)
    v = orc.randn(SEED_V + cfg, (nkeys, Hkv * D), sigma)
    kc, vc = orc.kv_store(kt, k, v, Hkv, D, cap, 0)
    if pm:
        kc = np.ascontiguousarray(kc.transpose(1, 0, 2))
        vc = np.ascontiguousarray(vc.transpose(1, 0, 2))
    return kc, vc


def make_q(qt, T, Hq, D, cfg=0, sigma=1.0):
    """Query rows: (what goes to the GPU, the same values as float32 for the oracle)."""
    q = orc.randn(SEED_Q + cfg, (T, Hq * D), sigma)
    if qt == F32:
        return q, q
    if qt == F16:
        b = orc.f2h(q)
        return b, orc.h2f(b)
    b = orc.f2bf(q)
    return b, orc.bf2f(b)


def out_dtype(qt):
    return np.float32 if qt == F32 else np.uint16


def out_to_f32(qt, raw):
    if qt == F32:
        return raw.astype(np.float32)
    return orc.h2f(raw) if qt == F16 else orc.bf2f(raw)


def gpu_decode(ops, qt, kt, q_dev_arr, kc, vc, T, Hq, Hkv, D, cap, p0, win=0, pm=False, scale=0.0, bufs=None):
    """One decode / verify pass on the GPU through ns_attn_decode_t; returns float32 [T][Hq*D]."""
    g = ops.gpu
    if bufs is None:
        bufs = (DevBuf.of(g, kc), DevBuf.of(g, vc))
    kcb, vcb = bufs
    qb = DevBuf.of(g, q_dev_arr)
    ob = DevBuf(g, T * Hq * D * (4 if qt == F32 else 2))
    ob.fill(0xFF)
    sc = DevBuf(g, max(4, 4 * ops.decode_scratch(T, Hq, Hkv, D, p0, win)))
    ops.decode(qt, kt, qb, Hq * D, kcb, vcb, T, Hq, Hkv, D, cap, p0, ob, sc, win=win, pm=pm, scale=scale)
    raw = ob.read(out_dtype(qt))
    return out_to_f32(qt, raw).reshape(T, Hq * D), raw


def gpu_prompt(ops, qt, kt, q_dev_arr, kc, vc, T, Hq, Hkv, D, cap, p0, win=0, pm=False, scale=0.0, bufs=None):
    g = ops.gpu
    if bufs is None:
        bufs = (DevBuf.of(g, kc), DevBuf.of(g, vc))
    kcb, vcb = bufs
    qb = DevBuf.of(g, q_dev_arr)
    ob = DevBuf(g, T * Hq * D * (4 if qt == F32 else 2))
    ob.fill(0xFF)
    ops.prompt(qt, kt, qb, Hq * D, kcb, vcb, T, Hq, Hkv, D, cap, p0, ob, win=win, pm=pm, scale=scale)
    raw = ob.read(out_dtype(qt))
    return out_to_f32(qt, raw).reshape(T, Hq * D), raw


def check_close(got, ref64, qt=F32, what="", kt=0):
    """The path's bar against the float64 closed form: max-abs 2e-3, relative L2 1e-3. Where bfloat16 enters - output
    rows of that type, or a bfloat16 cache (the kernel's MFMA operands are then bfloat16: the query and the softmax
    weights are rounded to 8 significant bits) - the bound of that rounding, 2^-9 relative, is added: a correctly
    rounded bfloat16 copy of the exact result already sits at ~1.6e-3 relative L2."""
    mx, rel, cos = orc.compare(got, ref64)
    tol_abs, tol_rel = MAX_ABS, REL_L2
    if qt == BF16 or kt == 3:
        # one rounding for the weights, one for an output of that type: each at most 2^-9 of the largest value
        tol_abs = MAX_ABS + ((qt == BF16) + (kt == 3)) * BF16_ROUND * float(np.abs(ref64).max())
        tol_rel = REL_L2 + BF16_ROUND
    assert np.isfinite(got).all(), "%s: non-finite output" % what
    assert mx <= tol_abs and rel <= tol_rel, "%s: max-abs %.3g (<= %.3g), rel-L2 %.3g (<= %.3g), cosine %.6f" % (what, mx, tol_abs, rel, tol_rel, cos)
    return mx, rel
