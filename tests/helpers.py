"""Shared by the parity tests: seeded inputs from the oracle's generator, caches packed by the oracle's stores, the
HIP path called through the C ABI wrappers, and the comparison measures (max-abs, relative L2) with the tolerances of
the path: max-abs 2e-3 and relative L2 1e-3 against the float64 closed form (`tolerances` states the one rule by which
the absolute bound grows with the output's size and a bfloat16 rounding widens both)."""
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


U_HALF, U_BF16 = 2.0 ** -11, 2.0 ** -8      # unit roundoffs: half carries 11 significant bits, bfloat16 8


def tolerances(ref64, qt=F32, kt=0):
    """The path's bar against the float64 closed form, as ONE rule for every cache form and row type.

    relative L2 <= 1e-3 and max-abs <= max(2e-3, sum of u |ref|max over the 16-bit roundings between the stored values
    and the output), u the unit roundoff of the rounded type (half 2^-11, bfloat16 2^-8). The roundings of a pass:
      - the softmax weights, rounded for the second product: half (the reference: qwen35/silo/attn.cpp:225-227) - also
        over a bfloat16 cache, whose values are widened to half for it (prompt passes) or whose weights are split into two
        bfloat16 numbers, 16 significant bits between them (decode passes, and prompt passes over a cache too long for the
        library's scratch to hold widened);
      - q8_0 / q4_0 values, staged as halfs before the products as the reference stages them (silo/attn.cpp:56-76), where
        the closed form multiplies the unrounded int x scale;
      - a 16-bit output row.
    Why max-abs scales with |ref|max: an output that is the mean of two values v1, v2 under weights rounded with unit
    roundoff u moves by up to u |v1 - v2| / 2 <= u |v|max, so the absolute bound 2e-3 can hold only while |out| < 4 (half).
    A bfloat16 rounding is 8 times coarser: each adds 2^-9 to the relative bound as well (a correctly rounded bfloat16
    copy of the exact result sits at ~1.6e-3 relative L2). Float32 / half query rows against bfloat16 operands
    enter the first product as two bfloat16 numbers (the rounded row and the rounded rest) and add no rounding of their own."""
    n_half = 1 + (kt in (1, 2)) + (qt == F16)
    n_bf16 = int(qt == BF16)
    big = float(np.abs(ref64).max())
    return max(MAX_ABS, (n_half * U_HALF + n_bf16 * U_BF16) * big), REL_L2 + n_bf16 * BF16_ROUND


def check_close(got, ref64, qt=F32, what="", kt=0):
    """got against the float64 closed form under `tolerances`; returns (max-abs, relative L2)."""
    mx, rel, cos = orc.compare(got, ref64)
    tol_abs, tol_rel = tolerances(ref64, qt, kt)
    assert np.isfinite(got).all(), "%s: non-finite output" % what
    assert mx <= tol_abs and rel <= tol_rel, "%s: max-abs %.3g (<= %.3g), rel-L2 %.3g (<= %.3g), cosine %.6f" % (what, mx, tol_abs, rel, tol_rel, cos)
    return mx, rel


def assert_bf16_rows_follow(raw16, got32, what=""):
    """A pass's bfloat16 output rows against the same pass's float32 output rows: each the rounding of the other's value up
    to the one bfloat16 step by which two roundings of nearly the same number may differ (bfloat16 query rows enter the
    first product as bfloat16, float32 ones as half: the same exact products, summed by two different matrix instructions),
    and the same number in all but a few per thousand."""
    want = orc.f2bf(np.ascontiguousarray(got32, np.float32)).ravel().astype(np.int32)
    have = np.asarray(raw16).ravel().astype(np.int32)
    step = np.abs(want - have)
    assert step.max() <= 1 and np.count_nonzero(step) <= 5e-3 * step.size, "%s: up to %d steps apart, %d of %d differ" % (what, step.max(), np.count_nonzero(step), step.size)
