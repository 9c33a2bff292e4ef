"""The HIP path against the committed golden fixtures (tests/golden/*.npz: inputs, expected cache bytes and float64 results
written from the definitions in numpy): the store kernels' bytes bit for bit, decode and prompt passes within the path's
tolerance, the absorbed MLA decode and GLM's q8 rows."""
import os

import numpy as np
import pytest

from helpers import check_close, gpu_decode, gpu_prompt
from nextsycl_amd import DevBuf
from nextsycl_amd.attn import BF16, F16, F32

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.mark.parametrize("kt", [0, 1, 2, 3])
@pytest.mark.parametrize("case", ["decode", "verify", "window", "prompt", "wide"])
def test_store_and_attention_on_the_fixtures(ops, case, kt):
    z = np.load(os.path.join(GOLD, "attention.npz"), allow_pickle=False)
    T, Hq, Hkv, D, p0, win = (int(x) for x in z[case + "_shape"])
    cap = p0 + T
    g = ops.gpu
    want_k, want_v = z["%s_kc%d" % (case, kt)], z["%s_vc%d" % (case, kt)]
    kc, vc = DevBuf(g, want_k.nbytes), DevBuf(g, want_v.nbytes)
    ops.kv_store(kt, DevBuf.of(g, z[case + "_k"]), Hkv * D, DevBuf.of(g, z[case + "_v"]), Hkv * D, cap, Hkv, D, cap, 0, kc, vc)
    assert np.array_equal(kc.read(np.uint8), want_k.ravel()) and np.array_equal(vc.read(np.uint8), want_v.ravel())
    q = z[case + "_q"]                                            # exact in half
    qt = BF16 if kt == 3 else F16
    qd = q.astype(np.float16).view(np.uint16)
    if kt == 3:
        # the fixture's bfloat16 result is for the queries rounded to bfloat16 (round to nearest even)
        u = q.view(np.uint32)
        qd = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    run = gpu_decode if T <= 16 else gpu_prompt
    got, _ = run(ops, qt, kt, qd, want_k, want_v, T, Hq, Hkv, D, cap, p0, win=win, bufs=(kc, vc))
    check_close(got, z["%s_out%d" % (case, kt)], qt, "fixture %s, cache form %d" % (case, kt), kt=kt)
    if T > 16:
        got32, _ = gpu_prompt(ops, F32, kt, q if kt != 3 else (qd.astype(np.uint32) << 16).view(np.float32), want_k, want_v, T, Hq, Hkv, D, cap, p0, win=win, bufs=(kc, vc))
        check_close(got32, z["%s_out%d" % (case, kt)], F32, "fixture %s, float32 rows" % case, kt=kt)


def test_mla_and_glm_rows_on_the_fixtures(ops):
    z = np.load(os.path.join(GOLD, "mla.npz"), allow_pickle=False)
    T, H, pos0 = (int(x) for x in z["shape"])
    g = ops.gpu
    ub = DevBuf(g, T * H * 512 * 4)
    ub.fill(0xFF)
    sc = DevBuf(g, 4 * ops.mla_latent_scratch(T, H, pos0))
    ops.mla_decode_latent(F32, DevBuf.of(g, z["qa"]), DevBuf.of(g, z["cache"]), ub, T, H, 64, pos0, float(z["scale"][0]), sc)
    check_close(ub.read(np.float32).reshape(T, H * 512), z["u"].reshape(T, H * 512), F32, "fixture MLA")
    rows = z["glm_rows"]
    yb = DevBuf(g, rows.nbytes)
    ops.to_q8row(DevBuf.of(g, z["glm_x"]), yb, rows.shape[0], 512)
    assert np.array_equal(yb.read(np.uint8).reshape(rows.shape), rows)


def test_rope_and_indexer_on_the_fixtures(ops):
    z = np.load(os.path.join(GOLD, "select.npz"), allow_pickle=False)
    g = ops.gpu
    T, H, head, off, n_dims, pos0 = (int(x) for x in z["rope_shape"])
    xb = DevBuf.of(g, z["rope_x"])
    ops.ok(ops.k.ds2_rope(ops.raw(), xb.ptr, T, H, H * head, head, off, n_dims, pos0, *(float(v) for v in z["rope_yarn"]), None, 0, 0), "ns_ds2_rope")
    assert np.abs(xb.read(np.float32).reshape(T, H * head) - z["rope_y"]).max() < 1e-4 * np.abs(z["rope_x"]).max() * float(z["rope_yarn"][3])
    D, n_tok, hh, K, Tq, q0 = (int(x) for x in z["idx_shape"])
    rb, pb, ab = DevBuf(g, 8 * 2 * D * 4), DevBuf(g, (n_tok // 4) * D * 4), DevBuf.of(g, z["idx_ape"])
    rb.fill(0)
    pb.fill(0)
    pos = 0
    for t in (30, 1, 2, 5, 12):
        kb, gb = DevBuf.of(g, z["idx_ik"][pos:pos + t]), DevBuf.of(g, z["idx_ig"][pos:pos + t])
        ops.ok(ops.k.idx_pool(ops.raw(), rb.ptr, kb.ptr, gb.ptr, ab.ptr, pb.ptr, pos, t, D), "ns_idx_pool")
        pos += t
    assert np.abs(pb.read(np.float32).reshape(-1, D) - z["idx_pooled"]).max() < 1e-5
    npool = n_tok // 4
    Sb, wb, scb = DevBuf.of(g, z["idx_S"]), DevBuf.of(g, z["idx_w"]), DevBuf(g, Tq * npool * 4)
    ops.ok(ops.k.idx_score(ops.raw(), Sb.ptr, wb.ptr, scb.ptr, Tq, hh, 0, npool, npool, q0), "ns_idx_score")
    score, want = scb.read(np.float32).reshape(Tq, npool), z["idx_score"]
    assert np.array_equal(np.isneginf(score), np.isneginf(want))
    assert np.abs(score[np.isfinite(want)] - want[np.isfinite(want)]).max() < 1e-5
    s32, selb = DevBuf.of(g, z["idx_score32"]), DevBuf.of(g, np.full((Tq, K), -1, np.int32))
    ops.ok(ops.k.topk(ops.raw(), s32.ptr, selb.ptr, Tq, npool, npool, K), "ns_topk")
    assert np.array_equal(selb.read(np.int32).reshape(Tq, K), z["idx_sel"])
