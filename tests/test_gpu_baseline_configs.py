"""BASELINE.json's configurations at their full sizes, through the C ABI, against the oracle: the decode-side ones
(configs 1, 3, 5 and the 32K target) in full against the float64 closed form; the 8192-row prefill (config 2) on three
whole 256-row blocks against the closed form plus size-independent properties over the whole output."""
import numpy as np
import pytest

from helpers import SEED_K, SEED_Q, SEED_V, assert_bf16_rows_follow, check_close, gpu_decode, gpu_prompt, make_kv, make_q
from nextsycl_amd import DevBuf
from nextsycl_amd.attn import BF16, F16, F32
from oracle import orc

pytestmark = pytest.mark.gpu


def test_config1_gqa_decode_4k(ops):
    """configs[0]: batch 1, 1 query token, 32 / 8 heads, head 128, KV 4096, f16, scale 1/sqrt(128); out f16 [32,128]."""
    T, Hq, Hkv, D, kv = 1, 32, 8, 128, 4096
    kc, vc = make_kv(0, Hkv, D, kv, kv, cfg=1)
    qd, qf = make_q(F16, T, Hq, D, cfg=1)
    got, raw = gpu_decode(ops, F16, 0, qd, kc, vc, T, Hq, Hkv, D, kv, kv - T)
    ref = orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, kv, kv - T)
    check_close(got, ref, F16, "config 1")
    assert raw.shape == (32 * 128,)
    # the reference's exact kernel (restated, float32) lands on the same closed form
    check_close(orc.attn_exact(qf, kc, vc, 0, T, Hq, Hkv, D, kv, kv - T), ref, F32, "config 1, exact restatement")


def test_decode_32k_target(ops):
    T, Hq, Hkv, D, kv = 1, 32, 8, 128, 32768
    kc, vc = make_kv(0, Hkv, D, kv, kv, cfg=6)
    qd, qf = make_q(F16, T, Hq, D, cfg=6)
    got, _ = gpu_decode(ops, F16, 0, qd, kc, vc, T, Hq, Hkv, D, kv, kv - T)
    check_close(got, orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, kv, kv - T), F16, "32K decode")


def test_config3_q8_0_decode_128k(ops):
    """configs[2]: q8_0 cache (rows of 136 bytes) of 131072 keys, 64 / 4 heads, head 128; the cache is written by the
    library's store kernel from float32 N(0,1) rows and must equal the oracle's bytes before it is attended."""
    T, Hq, Hkv, D, kv = 1, 64, 4, 128, 131072
    g = ops.gpu
    k = orc.randn(SEED_K + 3, (kv, Hkv * D))
    v = orc.randn(SEED_V + 3, (kv, Hkv * D))
    kc_ref, vc_ref = orc.kv_store(1, k, v, Hkv, D, kv, 0)
    assert kc_ref.shape == (4, 131072, 136)
    kc, vc = DevBuf(g, kc_ref.nbytes), DevBuf(g, vc_ref.nbytes)
    step = 16384
    for s in range(0, kv, step):
        ops.kv_store(1, DevBuf.of(g, k[s:s + step]), Hkv * D, DevBuf.of(g, v[s:s + step]), Hkv * D, step, Hkv, D, kv, s, kc, vc)
    assert np.array_equal(kc.read(np.uint8), kc_ref.ravel()) and np.array_equal(vc.read(np.uint8), vc_ref.ravel())
    qd, qf = make_q(F16, T, Hq, D, cfg=3)
    got, _ = gpu_decode(ops, F16, 1, qd, kc_ref, vc_ref, T, Hq, Hkv, D, kv, kv - T, bufs=(kc, vc))
    check_close(got, orc.attn_f64(qf, kc_ref, vc_ref, 1, T, Hq, Hkv, D, kv, kv - T), F16, "config 3")


def test_config5_mtp_verify_64k(ops):
    """configs[4]: 4 draft rows appended to a 65536-token cache, 32 / 4 heads, causal among the 4; and each row equals
    its own one-row decode bit for bit (multi-token reuse of the key tiles changes no row's arithmetic)."""
    T, Hq, Hkv, D, p0 = 4, 32, 4, 128, 65536
    cap = p0 + T
    kc, vc = make_kv(0, Hkv, D, cap, cap, cfg=5)
    qd, qf = make_q(F16, T, Hq, D, cfg=5)
    g = ops.gpu
    bufs = (DevBuf.of(g, kc), DevBuf.of(g, vc))
    got, raw = gpu_decode(ops, F16, 0, qd, kc, vc, T, Hq, Hkv, D, cap, p0, bufs=bufs)
    check_close(got, orc.attn_f64(qf, kc, vc, 0, T, Hq, Hkv, D, cap, p0), F16, "config 5")
    raw = raw.reshape(T, -1)
    for t in range(T):
        _, one = gpu_decode(ops, F16, 0, qd[t:t + 1], kc, vc, 1, Hq, Hkv, D, cap, p0 + t, bufs=bufs)
        assert np.array_equal(one, raw[t]), t


def test_config2_prefill_8k(ops, record_property):
    """configs[1]: seq 8192, 40 / 8 heads (G = 5), head 128, bf16 Q / K / V and output, causal. Three whole 256-row blocks
    (the first, a middle one, the last: every wave and row tile of a work-group, every head) against the float64 closed
    form, plus size-independent properties over the whole output."""
    T, Hq, Hkv, D = 8192, 40, 8, 128
    g = ops.gpu
    kc, vc = make_kv(3, Hkv, D, T, T, cfg=2)
    qd, qf = make_q(BF16, T, Hq, D, cfg=2)
    bufs = (DevBuf.of(g, kc), DevBuf.of(g, vc))
    got, raw = gpu_prompt(ops, BF16, 3, qd, kc, vc, T, Hq, Hkv, D, T, 0, bufs=bufs)
    assert np.isfinite(got).all() and raw.shape == (T * Hq * D,)
    # the float32-output variant of the same pass: the kernel's own error without the output's bfloat16 rounding, held to
    # the path's plain bar - max-abs 2e-3, relative L2 1e-3 (the cache's values are widened to half, exactly, and the
    # softmax weights are half); the bfloat16 output is its rounding
    got32, _ = gpu_prompt(ops, F32, 3, qf, kc, vc, T, Hq, Hkv, D, T, 0, bufs=bufs)
    assert_bf16_rows_follow(raw, got32, "config 2")
    worst = [0.0, 0.0]
    for r0 in (0, 4096, 7936):
        ref = orc.attn_f64(qf[r0:r0 + 256], kc, vc, 3, 256, Hq, Hkv, D, T, r0)
        check_close(got[r0:r0 + 256], ref, BF16, "config 2, rows %d.." % r0, kt=3)
        mx, rel, _ = orc.compare(got32[r0:r0 + 256], ref)
        print("config 2, float32 output, rows %d..%d: max-abs %.3e, relative L2 %.3e" % (r0, r0 + 255, mx, rel))
        worst = [max(worst[0], mx), max(worst[1], rel)]
        assert rel <= 1e-3 and mx <= 2e-3, (r0, mx, rel)
    record_property("config2_f32_max_abs", worst[0])
    record_property("config2_f32_rel_l2", worst[1])
    # row 0 sees one key: its output is that key's value row, exactly
    V0 = orc.kv_dequant(vc[:, 0], 3, D)            # [Hkv][D]
    assert np.array_equal(got[0].reshape(Hq, D), np.repeat(V0, Hq // Hkv, axis=0))
    # V = 1 everywhere: every one of the 8192 x 40 x 128 outputs is 1 (each row's weights sum to one)
    ones = np.ascontiguousarray(np.broadcast_to(np.array([0x3F80], np.uint16).view(np.uint8), (Hkv, T, D, 2)).reshape(Hkv, T, 2 * D))
    g1, _ = gpu_prompt(ops, F32, 3, qf, kc, ones, T, Hq, Hkv, D, T, 0, bufs=(bufs[0], DevBuf.of(g, ones)))
    assert np.abs(g1 - 1.0).max() < 1e-5         # numerator and denominator carry the very same rounded weights


def test_decode_and_prompt_at_256k_context(ops, tune):
    """The reference's long-context target (docs/256k-context.md): 262144 tokens in a q8_0 cache of 272-byte rows (heads
    of 256). A two-row verify pass and a 17-row prompt chunk at the cache's end against the float64 closed form; the
    prompt pass once over rows widened to half in the library's scratch (512 MiB of them) and once - with a quarter of
    the scratch to plan with - over the rows' own form, the way of a context too long to widen."""
    Hq, Hkv, D, n = 8, 2, 256, 262144
    kc, vc = make_kv(1, Hkv, D, n, n, cfg=1)
    assert kc.nbytes == Hkv * n * 272 and 2 * Hkv * n * D * 2 > 256 << 20
    g = ops.gpu
    bufs = (DevBuf.of(g, kc), DevBuf.of(g, vc))
    T = 2
    qd, qf = make_q(F16, T, Hq, D, cfg=4)
    got, _ = gpu_decode(ops, F16, 1, qd, kc, vc, T, Hq, Hkv, D, n, n - T, bufs=bufs)
    check_close(got, orc.attn_f64(qf, kc, vc, 1, T, Hq, Hkv, D, n, n - T), F16, "verify pass at 262144 keys", kt=1)
    T = 17
    qd, qf = make_q(F32, T, Hq, D, cfg=5)
    ref = orc.attn_f64(qf, kc, vc, 1, T, Hq, Hkv, D, n, n - T)
    got, _ = gpu_prompt(ops, F32, 1, qd, kc, vc, T, Hq, Hkv, D, n, n - T, bufs=bufs)
    check_close(got, ref, F32, "prompt chunk at 262144 keys, rows widened", kt=1)
    tune(6, 256)
    own, _ = gpu_prompt(ops, F32, 1, qd, kc, vc, T, Hq, Hkv, D, n, n - T, bufs=bufs)
    check_close(own, ref, F32, "prompt chunk at 262144 keys, the rows' own form", kt=1)
    assert np.array_equal(got, own)
