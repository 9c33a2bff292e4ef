"""Parity of the MLA path (include/ns_mla.h) against the oracle, through the C ABI: the absorbed latent decode
(BASELINE's MLA configuration), DeepSeek's full decode call, the latent cache store, GLM's latent-only form and q8 rows."""
import numpy as np
import pytest

from helpers import MAX_ABS, REL_L2
from nextsycl_amd import DevBuf, Error
from nextsycl_amd.attn import F16, F32
from oracle import orc

pytestmark = pytest.mark.gpu


def _latent(ops, qt, qa_dev, cache, T, H, R, pos0, scale):
    g = ops.gpu
    ub = DevBuf(g, T * H * 512 * (4 if qt == F32 else 2))
    ub.fill(0xFF)
    sc = DevBuf(g, 4 * ops.mla_latent_scratch(T, H, pos0))
    ops.mla_decode_latent(qt, DevBuf.of(g, qa_dev), DevBuf.of(g, cache), ub, T, H, R, pos0, scale, sc)
    raw = ub.read(np.float32 if qt == F32 else np.uint16)
    return (raw if qt == F32 else orc.h2f(raw)).reshape(T, H, 512)


def _close(got, ref, what):
    mx, rel, cos = orc.compare(got, ref)
    assert np.isfinite(got).all(), what
    assert mx <= MAX_ABS and rel <= REL_L2, "%s: max-abs %.3g, rel-L2 %.3g, cosine %.6f" % (what, mx, rel, cos)


@pytest.mark.parametrize("T,H,R,pos0,qt", [
    (1, 16, 64, 0, F32), (1, 128, 64, 31, F32), (1, 128, 64, 32, F16), (2, 128, 64, 700, F32), (8, 16, 64, 1000, F16),
    (1, 20, 64, 3000, F32), (3, 64, 0, 500, F32), (1, 128, 0, 2047, F16), (16, 128, 64, 100, F32)])
def test_latent_decode_small(ops, T, H, R, pos0, qt):
    n = pos0 + T
    cache = orc.f2h(orc.randn(1, (n, 512 + R), 0.5))
    qa = orc.randn(2, (T, H, 512 + R))
    scale = 1.0 / np.sqrt(192.0)
    qd, qf = (qa, qa) if qt == F32 else (orc.f2h(qa), orc.h2f(orc.f2h(qa)))
    got = _latent(ops, qt, qd, cache, T, H, R, pos0, scale)
    ref = orc.mla_f64(qf, cache, T, H, pos0, scale, 512, R)
    _close(got, ref, "latent decode vs float64 closed form")
    if R == 64:
        # the reference's kernel order (16 streams, exp), restated
        _close(orc.mla_decode_u(qf, cache, T, H, pos0, scale), ref, "the restatement itself")


@pytest.mark.parametrize("T,H,pos0,qt", [(1, 16, 49999, F32), (2, 32, 100000, F16), (1, 16, 131071, F16), (1, 16, 131072, F32),
                                         # 3 and 5 row groups: split counts chosen so that an XCD's places take whole splits
                                         (5, 64, 12000, F32), (5, 128, 6000, F16)])
def test_latent_decode_long_contexts(ops, T, H, pos0, qt):
    """One or two rows behind long contexts: the passes either side of the cell count at which the kernel's 64-row form
    gives way to the 128-row one, many tiles a split."""
    n = pos0 + T
    cache = orc.f2h(orc.randn(21, (n, 576), 0.5))
    qa = orc.randn(22, (T, H, 576))
    scale = 1.0 / np.sqrt(192.0)
    qd, qf = (qa, qa) if qt == F32 else (orc.f2h(qa), orc.h2f(orc.f2h(qa)))
    got = _latent(ops, qt, qd, cache, T, H, 64, pos0, scale)
    _close(got, orc.mla_f64(qf, cache, T, H, pos0, scale, 512, 64), "latent decode vs float64 closed form")


def _random_cases(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        T = int(rng.choice([1, 1, 2, 4, 7, 16]))
        H = int(rng.choice([1, 8, 16, 20, 64, 128]))
        R = int(rng.choice([64, 64, 0]))
        pos0 = int(rng.choice([rng.integers(0, 40), rng.integers(40, 600), rng.integers(600, 5000)]))
        out.append((T, H, R, pos0, int(rng.choice([F32, F16]))))
    return out


@pytest.mark.parametrize("T,H,R,pos0,qt", _random_cases(24, 20240609))
def test_latent_decode_seeded_shapes(ops, T, H, R, pos0, qt):
    n = pos0 + T
    cache = orc.f2h(orc.randn(5 + pos0 % 3, (n, 512 + R), 0.5))
    qa = orc.randn(6 + T, (T, H, 512 + R))
    scale = 1.0 / np.sqrt(192.0)
    qd, qf = (qa, qa) if qt == F32 else (orc.f2h(qa), orc.h2f(orc.f2h(qa)))
    got = _latent(ops, qt, qd, cache, T, H, R, pos0, scale)
    _close(got, orc.mla_f64(qf, cache, T, H, pos0, scale, 512, R), "latent decode vs float64 closed form")


@pytest.mark.parametrize("T,H,R,pos0,qt", [(40, 16, 64, 100, F16), (33, 128, 64, 0, F32), (17, 8, 0, 2000, F32), (64, 20, 64, 37, F16),
                                            (300, 16, 64, 250, F16), (1100, 8, 64, 0, F32), (70, 16, 0, 5000, F32), (300, 4, 64, 1900, F16),
                                            # 20 and 23 row groups behind 4096 cells and more: cut at 16 groups, the rest a pass of its own
                                            (20, 128, 64, 4500, F16), (45, 64, 0, 6000, F32)])
def test_latent_prompt_widths(ops, T, H, R, pos0, qt):
    """A prompt's rows through the same entry point (the reference's GEMM chain + masked softmax over these rows:
    llm/deepseek2/src/engine.rs:1165-1253): row t over cells 0 .. pos0 + t, against the float64 closed form. The passes
    are 128 rows, 256 behind long enough contexts, and end at 16 row groups where 17 to 27 would follow: the cases cross
    all of these."""
    n = pos0 + T
    cache = orc.f2h(orc.randn(9, (n, 512 + R), 0.5))
    qa = orc.randn(10, (T, H, 512 + R))
    scale = 1.0 / np.sqrt(192.0)
    qd, qf = (qa, qa) if qt == F32 else (orc.f2h(qa), orc.h2f(orc.f2h(qa)))
    got = _latent(ops, qt, qd, cache, T, H, R, pos0, scale)
    _close(got, orc.mla_f64(qf, cache, T, H, pos0, scale, 512, R), "prompt rows vs float64 closed form")
    # split anywhere, the rows are the same within the tolerance (another pass width sums in another order)
    lo = T // 2
    alone = _latent(ops, qt, qd[lo:], cache, T - lo, H, R, pos0 + lo, scale)
    _close(alone, got[lo:], "the second half on its own")


def test_prompt_chunk_at_bench_size(ops):
    """bench.py's `mla_prompt8k` at its full size (256 rows behind 8192 cells, 128 heads, half rows): the first and the
    last row against the float64 closed form, and the last 16 rows against the same rows as a decode-width pass of their
    own (another pass width, another summation order: within the tolerance)."""
    g = ops.gpu
    T, H, R, pos0 = 256, 128, 64, 8192
    n = pos0 + T
    scale = 1.0 / np.sqrt(192.0)
    cache = orc.f2h(orc.randn(21, (n, 512 + R), 0.5))
    qa = orc.f2h(orc.randn(22, (T, H, 512 + R)))
    got = _latent(ops, F16, qa, cache, T, H, R, pos0, scale)
    qf = orc.h2f(qa)
    for t in (0, T - 1):
        ref = orc.mla_f64(qf[t:t + 1], cache[:pos0 + t + 1], 1, H, pos0 + t, scale, 512, R)
        _close(got[t:t + 1], ref, "row %d vs float64 closed form" % t)
    lo = T - 16
    alone = _latent(ops, F16, qa[lo:], cache, 16, H, R, pos0 + lo, scale)
    _close(alone, got[lo:], "the last 16 rows as a pass of their own")


def test_config4_mla_decode_32k(ops):
    """BASELINE configs[3]: 128 heads, 512 latent + 64 rope, latent cache f16 ~N(0, 0.5), absorbed q of 576 a head,
    KV length 32768, scale 1/sqrt(192); output the 512-d latent a head, f16."""
    T, H, R, n = 1, 128, 64, 32768
    cache = orc.f2h(orc.randn(0xB0B + 4, (n, 576), 0.5))
    qa = orc.randn(0xA11CE + 4, (T, H, 576))
    qh = orc.f2h(qa)
    scale = 1.0 / np.sqrt(192.0)
    got = _latent(ops, F16, qh, cache, T, H, R, n - 1, scale)
    ref = orc.mla_f64(orc.h2f(qh), cache, T, H, n - 1, scale, 512, R)
    _close(got, ref, "config 4")


def test_full_ds2_mla_decode(ops):
    """ns_ds2_mla_decode: absorb (k_b), latent decode, value up-projection (v_b), as the engine calls it
    (llm/deepseek2/src/engine.rs:1150-1163)."""
    T, H, pos0 = 2, 16, 600
    n = pos0 + T
    g = ops.gpu
    cache = orc.f2h(orc.randn(1, (n, 576), 0.5))
    q = orc.randn(2, (T, H, 192))
    kb = orc.f2h(orc.randn(3, (H, 512, 128), 0.09))
    vb = orc.f2h(orc.randn(4, (H, 128, 512), 0.05))
    scale = 0.0722
    out = DevBuf(g, T * H * 128 * 4)
    ops.mla_decode(DevBuf.of(g, q), DevBuf.of(g, kb), DevBuf.of(g, vb), DevBuf.of(g, cache), out, T, H, pos0, scale)
    got = out.read(np.float32).reshape(T, H, 128)
    qa = orc.mla_absorb(q, kb, T, H)
    u = orc.mla_decode_u(qa, cache, T, H, pos0, scale)
    want = orc.mla_vb(u, vb, T, H)
    # float64 end to end
    qa64 = np.concatenate([np.einsum("hrc,thc->thr", orc.h2f(kb).astype(np.float64), q[:, :, :128].astype(np.float64)), q[:, :, 128:]], axis=2)
    u64 = orc.mla_f64(qa64.astype(np.float32), cache, T, H, pos0, scale)
    want64 = np.einsum("hvl,thl->thv", orc.h2f(vb).astype(np.float64), u64)
    _close(got, want64, "ns_ds2_mla_decode vs float64")
    _close(want, want64, "the restated chain itself")


def test_full_ds2_mla_decode_of_more_rows_than_a_pass(ops):
    """ns_ds2_mla_decode takes any row count, as the reference's kernel does (kernels/llm/deepseek2/ds2.cpp:262-270): 41
    rows are three queued passes, every row at its own position."""
    T, H, pos0 = 41, 8, 250
    n = pos0 + T
    g = ops.gpu
    cache = orc.f2h(orc.randn(5, (n, 576), 0.5))
    q = orc.randn(6, (T, H, 192))
    kb = orc.f2h(orc.randn(7, (H, 512, 128), 0.09))
    vb = orc.f2h(orc.randn(8, (H, 128, 512), 0.05))
    scale = 0.0722
    out = DevBuf(g, T * H * 128 * 4)
    out.fill(0xFF)
    ops.mla_decode(DevBuf.of(g, q), DevBuf.of(g, kb), DevBuf.of(g, vb), DevBuf.of(g, cache), out, T, H, pos0, scale)
    got = out.read(np.float32).reshape(T, H, 128)
    qa64 = np.concatenate([np.einsum("hrc,thc->thr", orc.h2f(kb).astype(np.float64), q[:, :, :128].astype(np.float64)), q[:, :, 128:]], axis=2)
    u64 = orc.mla_f64(qa64.astype(np.float32), cache, T, H, pos0, scale)
    _close(got, np.einsum("hvl,thl->thv", orc.h2f(vb).astype(np.float64), u64), "ns_ds2_mla_decode, 41 rows")


def test_ds2_kv_store(ops):
    g = ops.gpu
    T, L, R, pos0 = 37, 512, 64, 40
    kv = orc.randn(1, (T, L + R))
    w = orc.randn(2, (L,), 0.3) + 1.0
    for yarn in ((10000.0, 1.0, 0.0, 1.0, 0.0, 0.0), (10000.0, 0.025, 1.0, 1.3, 10.0, 23.0)):
        want = np.zeros((pos0 + T, L + R), np.uint16)
        orc.ds2_kv_store(kv, w, 1e-6, want, T, L, R, pos0, *yarn)
        cb = DevBuf(g, want.nbytes)
        cb.fill(0)
        ops.ds2_kv_store(DevBuf.of(g, kv), DevBuf.of(g, w), 1e-6, cb, T, L, R, pos0, *yarn)
        got = cb.read(np.uint16).reshape(want.shape)
        assert (got[:pos0] == 0).all()
        # the normalized latent half has no library function in it (the sum of squares is taken in float64 on both sides,
        # the square root and the division are correctly rounded): bit for bit
        assert np.array_equal(got[pos0:, :L], want[pos0:, :L])
        # the rotated half: cos / sin come from another library, so a half may differ in its last bit
        gr, wr = orc.h2f(got[pos0:, L:]).astype(np.float64), orc.h2f(want[pos0:, L:]).astype(np.float64)
        assert (np.abs(gr - wr) <= np.abs(wr) * 2.0 ** -10 + 1e-6).all()
        assert (got[pos0:, L:] == want[pos0:, L:]).mean() > 0.9


@pytest.mark.parametrize("yarn", [(10000.0, 1.0, 0.0, 1.0, 0.0, 0.0), (10000.0, 0.025, 1.0, 1.3, 10.0, 23.0)])
def test_ds2_rope(ops, yarn):
    """ns_ds2_rope (kernels/llm/deepseek2/ds2.cpp:59-83): a decode step's q_pe - 64 of each head's 192 floats - turned in
    place, the copy to `out`, every other float untouched; cos / sin come from another library than the oracle's, so a
    float may differ by a few ulps of the angle."""
    T, H, head, off, n, pos0 = 7, 16, 192, 128, 64, 3000
    row = H * head + 5
    g = ops.gpu
    x = orc.randn(7, (T, row))
    want_out = np.zeros((T, H, n), np.float32)
    want = orc.ds2_rope(x.copy(), T, H, row, head, off, n, pos0, *yarn, want_out, H * n, n)
    xb, ob = DevBuf.of(g, x), DevBuf(g, want_out.nbytes)
    ob.fill(0)
    ops.ok(ops.k.ds2_rope(ops.raw(), xb.ptr, T, H, row, head, off, n, pos0, *yarn, ob.ptr, H * n, n), "ns_ds2_rope")
    got, got_out = xb.read(np.float32).reshape(T, row), ob.read(np.float32).reshape(T, H, n)
    rot = np.zeros((T, row), bool)
    for h in range(H):
        rot[:, h * head + off:h * head + off + n] = True
    assert np.array_equal(got[~rot], x[~rot])
    tol = (4.0 * (1.0 + pos0 + T) * 2.0 ** -23 + 2e-6) * float(np.abs(x).max()) * max(1.0, yarn[3])
    assert np.abs(got - want).max() <= tol and np.abs(got_out - want_out).max() <= tol
    assert np.array_equal(got_out.reshape(T, H * n), got[rot].reshape(T, H * n))
    # no copy asked for, and the refusal
    xb2 = DevBuf.of(g, x)
    ops.ok(ops.k.ds2_rope(ops.raw(), xb2.ptr, T, H, row, head, off, n, pos0, *yarn, None, 0, 0), "ns_ds2_rope")
    assert np.array_equal(xb2.read(np.float32).reshape(T, row), got)
    with pytest.raises(Error, match="an even rotated width"):
        ops.ok(ops.k.ds2_rope(ops.raw(), xb2.ptr, T, H, row, head, off, 63, pos0, *yarn, None, 0, 0), "ns_ds2_rope")


def test_full_ds2_mla_decode_at_bench_size(ops):
    """ns_ds2_mla_decode at the size its timing is quoted at: one row, 128 heads, 32768 cells; every head against the float64
    chain."""
    T, H, pos0 = 1, 128, 32767
    n = pos0 + T
    g = ops.gpu
    cache = orc.f2h(orc.randn(11, (n, 576), 0.5))
    q = orc.randn(12, (T, H, 192))
    kb = orc.f2h(orc.randn(13, (H, 512, 128), 0.09))
    vb = orc.f2h(orc.randn(14, (H, 128, 512), 0.05))
    scale = 1.0 / np.sqrt(192.0)
    out = DevBuf(g, T * H * 128 * 4)
    out.fill(0xFF)
    ops.mla_decode(DevBuf.of(g, q), DevBuf.of(g, kb), DevBuf.of(g, vb), DevBuf.of(g, cache), out, T, H, pos0, scale)
    got = out.read(np.float32).reshape(T, H, 128)
    qa64 = np.concatenate([np.einsum("hrc,thc->thr", orc.h2f(kb).astype(np.float64), q[:, :, :128].astype(np.float64)), q[:, :, 128:]], axis=2)
    u64 = orc.mla_f64(qa64.astype(np.float32), cache, T, H, pos0, scale)
    want64 = np.einsum("hvl,thl->thv", orc.h2f(vb).astype(np.float64), u64)
    _close(got, want64, "ns_ds2_mla_decode at 128 heads x 32768 cells vs float64")


def test_q8_latent_at_32k_cells(ops):
    """GLM's q8 latent rows at 32768 cells, 2 rows x 128 heads: against the float64 closed form over the widened rows."""
    T, H, L, pos0 = 2, 128, 512, 32766
    n = pos0 + T
    g = ops.gpu
    x = orc.randn(21, (n, L), 0.5)
    qa = orc.randn(22, (T, H, L))
    rows = orc.glm_to_q8row(x, L)
    yb = DevBuf(g, rows.nbytes)
    ops.to_q8row(DevBuf.of(g, x), yb, n, L)
    assert np.array_equal(yb.read(np.uint8).reshape(rows.shape), rows)
    u = DevBuf(g, T * H * L * 4)
    u.fill(0xFF)
    ops.mla_attend(DevBuf.of(g, qa), yb, u, T, H, L, pos0, 0.04, q8=True)
    # the rows as the kernel widens them: half(scale x q), one rounding
    d = orc.h2f(rows[:, :32].copy().view(np.uint16)).astype(np.float32)                      # [n][16]
    qv = rows[:, 32:].view(np.int8).astype(np.float32).reshape(n, 16, 32)
    wide = orc.f2h((d[:, :, None] * qv).reshape(n, L))
    _close(u.read(np.float32).reshape(T, H, L), orc.mla_f64(qa, wide, T, H, pos0, 0.04, L, 0), "q8 latent MLA at 32768 cells")


def test_glm_latent_only_and_q8_rows(ops):
    g = ops.gpu
    T, H, L, pos0 = 2, 64, 512, 1500
    n = pos0 + T
    x = orc.randn(1, (n, L), 0.5)
    qa = orc.randn(2, (T, H, L))
    half = orc.f2h(x)
    u = DevBuf(g, T * H * L * 4)
    ops.mla_attend(DevBuf.of(g, qa), DevBuf.of(g, half), u, T, H, L, pos0, 0.04)
    _close(u.read(np.float32).reshape(T, H, L), orc.mla_f64(qa, half, T, H, pos0, 0.04, L, 0), "GLM latent MLA")
    # q8 rows: written by the library, bit for bit the oracle's; then attended
    want_rows = orc.glm_to_q8row(x, L)
    yb = DevBuf(g, want_rows.nbytes)
    ops.to_q8row(DevBuf.of(g, x), yb, n, L)
    assert np.array_equal(yb.read(np.uint8).reshape(want_rows.shape), want_rows)
    ops.mla_attend(DevBuf.of(g, qa), yb, u, T, H, L, pos0, 0.04, q8=True)
    ref = orc.glm_mla_attend(qa, want_rows, True, T, H, L, pos0, 0.04)
    _close(u.read(np.float32).reshape(T, H, L), ref.astype(np.float64), "GLM q8 latent MLA vs the reference-order restatement")
    # pool counts without pools are rejected (pools without counts are a dense pass, as in the reference)
    assert ops.k.mla_attend_sel(g.raw, u.ptr, u.ptr, u.ptr, 1, 1, 512, 0, 1.0, None, u.ptr, 4) == -1
    assert "selection" in ops.k.api.error()
