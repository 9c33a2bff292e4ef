"""The half products an engine's MLA prompt chain calls - ns_to_f16, ns_gemm_f16, ns_gemm_batch_h (the reference: oneMKL,
kernels/llm/glm5next/glm.cpp:208-276) - through the C ABI.

What pins them: numpy's float64 product of the same half operands (a float32 sum of exact half x half products may differ
from it by the sum's own roundings only: at most K 2^-23 sum |x| |w| here), numpy's own float32 -> float16 rounding bit for
bit, and the chain itself - scores, masked softmax, weighted sum - against ns_mla_attend_sel on the same rows."""
import numpy as np
import pytest

from nextsycl_amd import DevBuf, Error
from oracle import orc

pytestmark = pytest.mark.gpu


def _half(seed, shape, s=1.0):
    return (orc.randn(seed, shape) * s).astype(np.float16)


def _bound(x, w_t, K):
    """the float32 sum's worst case against the exact product: every partial sum rounded once"""
    return (K + 2) * 2.0 ** -23 * (np.abs(x.astype(np.float64)) @ np.abs(w_t.astype(np.float64))) + 1e-30


def test_to_f16_is_numpys_rounding(ops):
    g = ops.gpu
    x = orc.randn(3, (100003,)).astype(np.float32) * 37.0
    # ties, the subnormal range, the overflow edge, signed zeros and infinities
    x[:12] = [0.0, -0.0, 65504.0, 65519.9, 65520.0, -70000.0, 6e-8, 2.98e-8, 2.9802322e-8, 1.0009765625, 1.00146484375, np.inf]
    x[12:2012] = (np.arange(2000, dtype=np.float32) + 0.5) * 2.0 ** -25           # halfway between subnormals
    for n, off in ((x.size, 0), (x.size - 1, 1), (3, 2), (1, 0), (0, 0)):
        xb = DevBuf.of(g, x)
        yb = DevBuf(g, max(2 * x.size, 2))
        yb.fill(0xEE)
        ops.to_f16(xb.view(4 * off, 4 * n) if n else xb, yb.view(2 * off, 2 * n) if n else yb, n)
        got = yb.read(np.uint16)
        with np.errstate(over="ignore"):
            want = x[off:off + n].astype(np.float16).view(np.uint16)
        assert np.array_equal(got[off:off + n], want), (n, off)
        assert (got[:off] == 0xEEEE).all() and (got[off + n:] == 0xEEEE).all()


# T, N, K, ldx extra, ldy extra: whole blocks, ragged edges in every dimension, a K below one step, strides that break the
# 16-byte loads, a single row and column
SHAPES = [(64, 64, 64, 0, 0), (128, 192, 512, 0, 0), (1, 1, 1, 0, 0), (7, 5, 3, 0, 0), (65, 63, 33, 0, 0), (100, 130, 260, 4, 3),
          (16, 512, 576, 8, 0), (333, 17, 1000, 1, 7), (2, 700, 8, 0, 0), (130, 64, 40, 24, 64),
          # the tiled form (whole stages of 64 in K, more than 128 rows): one block and many, ragged rows and columns, padded rows
          (100, 64, 64, 0, 0), (191, 200, 64, 8, 1), (192, 200, 64, 0, 0), (129, 64, 64, 0, 0), (256, 128, 128, 0, 0), (300, 200, 192, 8, 5), (1000, 129, 576, 0, 0), (2048, 520, 512, 16, 8)]


@pytest.mark.parametrize("T,N,K,px,py", SHAPES)
def test_gemm_f16_against_the_exact_product(ops, T, N, K, px, py):
    g = ops.gpu
    ldx, ldy = K + px, N + py
    x, w = _half(T + N, (T, ldx)), _half(K + 7, (N, K), 0.5)
    y0 = orc.randn(9, (T, ldy)).astype(np.float32)
    want = x[:, :K].astype(np.float64) @ w.astype(np.float64).T
    bound = _bound(x[:, :K], w.T, K)
    xb, wb = DevBuf.of(g, x), DevBuf.of(g, w)
    for acc in (False, True):
        yb = DevBuf.of(g, y0)
        ops.gemm_f16(T, N, K, xb, ldx, wb, yb, ldy, acc)
        got = yb.read(np.float32).reshape(T, ldy)
        assert np.array_equal(got[:, N:], y0[:, N:])                                # nothing beside the N columns is written
        ref = want + (y0[:, :N] if acc else 0.0)
        err = np.abs(got[:, :N] - ref)
        assert (err <= bound + (2.0 ** -23 * np.abs(ref) if acc else 0.0)).all(), (T, N, K, acc, err.max())


# batch, trans_w, T, N, K, pads of ldx / ldw / ldy, gaps of sx / sw / sy
BATCHES = [(4, 1, 16, 300, 512, 0, 0, 0, 0, 0, 0), (3, 0, 16, 512, 300, 0, 0, 0, 0, 0, 0), (5, 0, 33, 70, 45, 3, 5, 1, 7, 9, 11),
           (5, 1, 33, 70, 45, 3, 5, 1, 7, 9, 11), (64, 0, 8, 512, 64, 0, 0, 0, 0, 0, 0), (2, 0, 1, 1, 1, 0, 0, 0, 0, 0, 0),
           (1, 0, 200, 129, 31, 0, 8, 0, 0, 0, 0), (2, 0, 64, 64, 96, 8, 16, 0, 8, 16, 0),
           # the tiled form in both orientations: ragged blocks, columns that end inside a chunk's block, padded strides
           (2, 0, 300, 200, 192, 8, 8, 3, 8, 16, 5), (2, 1, 300, 200, 192, 8, 8, 3, 8, 16, 5), (1, 0, 1030, 512, 640, 0, 64, 0, 0, 0, 0),
           (3, 0, 257, 72, 64, 0, 0, 0, 0, 0, 0), (1, 1, 4100, 1088, 576, 0, 0, 0, 0, 0, 0),
           # a batch of rows, a product a row's heads (GLM's chain): 128-row blocks
           (5, 1, 64, 320, 512, 0, 0, 0, 0, 0, 0), (5, 0, 64, 512, 320, 0, 0, 0, 0, 0, 0), (3, 1, 96, 200, 256, 8, 8, 8, 8, 8, 8)]


@pytest.mark.parametrize("B,tw,T,N,K,px,pw,py,gx,gw,gy", BATCHES)
def test_gemm_batch_h_both_forms(ops, B, tw, T, N, K, px, pw, py, gx, gw, gy):
    g = ops.gpu
    ldx, ldy = K + px, N + py
    wr, wc = (N, K) if tw else (K, N)
    ldw = wc + pw
    sx, sw, sy = T * ldx + gx, wr * ldw + gw, T * ldy + gy
    x, w = _half(B + T, (B * sx,)), _half(B + N, (B * sw,), 0.5)
    y0 = orc.randn(11, (B * sy,)).astype(np.float32)
    xb, wb = DevBuf.of(g, x), DevBuf.of(g, w)
    for acc in (False, True):
        yb = DevBuf.of(g, y0)
        ops.gemm_batch_h(B, tw, T, N, K, xb, ldx, sx, wb, ldw, sw, yb, ldy, sy, acc)
        got = yb.read(np.float32)
        written = np.zeros(B * sy, bool)
        for b in range(B):
            xm = x[b * sx:b * sx + T * ldx].reshape(T, ldx)[:, :K]
            wm = w[b * sw:b * sw + wr * ldw].reshape(wr, ldw)[:, :wc]
            wt = wm.T if tw else wm
            ym = got[b * sy:b * sy + T * ldy].reshape(T, ldy)[:, :N]
            y0m = y0[b * sy:b * sy + T * ldy].reshape(T, ldy)[:, :N]
            ref = xm.astype(np.float64) @ wt.astype(np.float64) + (y0m if acc else 0.0)
            err = np.abs(ym - ref)
            assert (err <= _bound(xm, wt, K) + (2.0 ** -23 * np.abs(ref) if acc else 0.0)).all(), (b, acc, err.max())
            written[b * sy:b * sy + T * ldy].reshape(T, ldy)[:, :N] = True
        assert np.array_equal(got[~written], y0[~written])


def test_gemm_refusals_and_empty_products(ops):
    g = ops.gpu
    x, w = DevBuf.of(g, _half(1, (64, 64))), DevBuf.of(g, _half(2, (64, 64)))
    y0 = orc.randn(3, (64, 64)).astype(np.float32)
    y = DevBuf.of(g, y0)
    for T, N in ((0, 64), (64, 0)):
        ops.gemm_f16(T, N, 64, x, 64, w, y, 64)
        assert np.array_equal(y.read(np.float32).reshape(64, 64), y0)
    ops.gemm_batch_h(0, 1, 64, 64, 64, x, 64, 0, w, 64, 0, y, 64, 0)
    assert np.array_equal(y.read(np.float32).reshape(64, 64), y0)
    # K = 0: an empty sum - zeros, or y as it was
    ops.gemm_batch_h(1, 0, 64, 64, 0, x, 64, 0, w, 64, 0, y, 64, 0, True)
    assert np.array_equal(y.read(np.float32).reshape(64, 64), y0)
    ops.gemm_batch_h(1, 0, 64, 64, 0, x, 64, 0, w, 64, 0, y, 64, 0, False)
    assert not y.read(np.float32).any()
    k = ops.k
    with pytest.raises(Error, match="apart"):
        ops.ok(k.gemm_f16(ops.raw(), 64, 64, 64, x.ptr, 32, w.ptr, y.ptr, 64, 0), "gemm_f16")
    with pytest.raises(Error, match="apart"):
        ops.ok(k.gemm_batch_h(ops.raw(), 1, 0, 64, 64, 32, x.ptr, 64, 0, w.ptr, 32, 0, y.ptr, 64, 0, 0), "gemm_batch_h")
    with pytest.raises(Error, match="null"):
        ops.ok(k.gemm_f16(ops.raw(), 64, 64, 64, None, 64, w.ptr, y.ptr, 64, 0), "gemm_f16")


@pytest.mark.parametrize("T,H,pos0", [(16, 8, 1000), (40, 4, 0), (5, 64, 2300)])
def test_the_prompt_chain_agrees_with_the_fused_pass(ops, T, H, pos0):
    """An engine's prompt branch as the reference runs it (llm/glm5next: cells, half scores, masked softmax, half weighted
    sum) on this library's pieces, against ns_mla_attend_sel over the same rows."""
    g = ops.gpu
    L, n_cells, scale = 512, pos0 + T, 0.0442
    NC = (n_cells + 63) // 64 * 64
    qa = orc.randn(T * H + pos0, (T * H, L)).astype(np.float32)
    cache = np.zeros((NC, L), np.float16)
    cache[:n_cells] = _half(77 + pos0, (n_cells, L), 0.7)
    qb, cb = DevBuf.of(g, qa), DevBuf.of(g, cache)
    # the fused pass
    uf = DevBuf(g, T * H * L * 4)
    ops.mla_attend(qb, cb, uf, T, H, L, pos0, scale)
    fused = uf.read(np.float32).reshape(T * H, L)
    # the chain
    idx, cnt = DevBuf(g, T * NC * 4), DevBuf(g, T * 4)
    ops.mla_cells(T, 0, pos0, idx, cnt, NC)
    assert np.array_equal(cnt.read(np.int32), pos0 + 1 + np.arange(T))
    qh = DevBuf(g, T * H * L * 2)
    ops.to_f16(qb, qh, T * H * L)
    S = DevBuf(g, T * H * NC * 4)
    ops.gemm_batch_h(1, 1, T * H, NC, L, qh, L, 0, cb, L, 0, S, NC, 0)
    ops.softmax_masked(S, T, H, NC, cnt, scale)
    ph = DevBuf(g, T * H * NC * 2)
    ops.to_f16(S, ph, T * H * NC)
    uc = DevBuf(g, T * H * L * 4)
    uc.fill(0xFF)
    ops.gemm_batch_h(1, 0, T * H, L, NC, ph, NC, 0, cb, L, 0, uc, L, 0)
    chain = uc.read(np.float32).reshape(T * H, L)
    # both round the softmax weights to half once and sum in float32
    assert np.abs(chain - fused).max() <= 2e-3
    assert np.linalg.norm(chain - fused) <= 1e-3 * np.linalg.norm(fused)


@pytest.mark.parametrize("T,H,pos0", [(3, 16, 700), (24, 16, 1000), (40, 128, 90)])
def test_deepseek_prompt_branch_call_for_call(ops, T, H, pos0):
    """The DeepSeek engine's prompt / long-context branch as it calls the library (llm/deepseek2/src/engine.rs:1165-1253):
    queries to half, absorbed by k_b (a batch a row at decode widths, a product a head beyond), scores against the cache,
    masked softmax, the weights to half, the weighted sum over the cache's latent columns (rows 576 apart, 512 read), u to
    half, v_b - against the float64 chain, and against ns_ds2_mla_decode over the same inputs."""
    g = ops.gpu
    nope, rope, lat, vl = 128, 64, 512, 128
    kl, cr = nope + rope, lat + rope
    n = pos0 + T
    nc = (n + 63) // 64 * 64
    scale = 1.0 / np.sqrt(192.0)
    cache = np.zeros((nc, cr), np.uint16)
    cache[:n] = orc.f2h(orc.randn(31 + T, (n, cr), 0.5))
    q = orc.randn(32 + T, (T, H, kl))
    kb = orc.f2h(orc.randn(33, (H, lat, nope), 0.09))
    vb = orc.f2h(orc.randn(34, (H, vl, lat), 0.05))
    qd, kbd, vbd, cd = DevBuf.of(g, q), DevBuf.of(g, kb), DevBuf.of(g, vb), DevBuf.of(g, cache)
    # the rotated part sits in qf already (the engine's rope writes it there)
    qf_host = np.zeros((T, H, cr), np.float32)
    qf_host[:, :, lat:] = q[:, :, nope:]
    qf = DevBuf.of(g, qf_host)
    q16 = DevBuf(g, T * H * kl * 2)
    ops.to_f16(qd, q16, T * H * kl)
    sub = lambda b, at, esz: b.view(at * esz, b.len - at * esz)
    if T <= 8:
        for r in range(T):
            ops.gemm_batch_h(H, True, 1, lat, nope, sub(q16, r * H * kl, 2), kl, kl, kbd, nope, lat * nope, sub(qf, r * H * cr, 4), cr, cr)
    else:
        for hh in range(H):
            ops.gemm_f16(T, lat, nope, sub(q16, hh * kl, 2), H * kl, sub(kbd, hh * lat * nope, 2), sub(qf, hh * cr, 4), H * cr)
    qh = DevBuf(g, T * H * cr * 2)
    ops.to_f16(qf, qh, T * H * cr)
    sc = DevBuf(g, T * H * nc * 4)
    ops.gemm_f16(T * H, nc, cr, qh, cr, cd, sc, nc)
    cnt = DevBuf.of(g, (pos0 + 1 + np.arange(T)).astype(np.int32))
    ops.softmax_masked(sc, T, H, nc, cnt, scale)
    ph = DevBuf(g, T * H * nc * 2)
    ops.to_f16(sc, ph, T * H * nc)
    u = DevBuf(g, T * H * lat * 4)
    u.fill(0xFF)
    ops.gemm_batch_h(1, False, T * H, lat, nc, ph, nc, T * H * nc, cd, cr, nc * cr, u, lat, T * H * lat)
    uh = DevBuf(g, T * H * lat * 2)
    ops.to_f16(u, uh, T * H * lat)
    oh = DevBuf(g, T * H * vl * 4)
    oh.fill(0xFF)
    if T <= 8:
        for r in range(T):
            ops.gemm_batch_h(H, True, 1, vl, lat, sub(uh, r * H * lat, 2), lat, lat, vbd, lat, vl * lat, sub(oh, r * H * vl, 4), vl, vl)
    else:
        for hh in range(H):
            ops.gemm_f16(T, vl, lat, sub(uh, hh * lat, 2), H * lat, sub(vbd, hh * vl * lat, 2), sub(oh, hh * vl, 4), H * vl)
    chain = oh.read(np.float32).reshape(T, H * vl)
    # the float64 chain over the same stored values
    qa64 = np.concatenate([np.einsum("hrc,thc->thr", orc.h2f(kb).astype(np.float64), orc.h2f(orc.f2h(q[:, :, :nope])).astype(np.float64)), q[:, :, nope:]], axis=2)
    u64 = orc.mla_f64(qa64.astype(np.float32), cache[:n], T, H, pos0, scale)
    want = np.einsum("hvl,thl->thv", orc.h2f(vb).astype(np.float64), u64).reshape(T, H * vl)
    assert np.abs(chain - want).max() <= 2e-3 and np.linalg.norm(chain - want) <= 1e-3 * np.linalg.norm(want)
    # and the decode-width entry point over the same inputs (any row count: passes of 16 rows)
    fused = DevBuf(g, T * H * vl * 4)
    fused.fill(0xFF)
    ops.mla_decode(qd, kbd, vbd, DevBuf.of(g, cache[:n]), fused, T, H, pos0, scale)
    f = fused.read(np.float32).reshape(T, H * vl)
    assert np.abs(chain - f).max() <= 2e-3 and np.linalg.norm(chain - f) <= 1.5e-3 * np.linalg.norm(f)


def test_gemm_sweep(ops):
    """A hundred seeded products over what the two kernel forms branch on - rows, columns, depth, both forms of w, padded
    rows and gaps between the batch's matrices, aligned or not, adding to y or not - against the exact product; nothing
    beside the T x N results may change."""
    g = ops.gpu
    rng = np.random.default_rng(20250304)
    for it in range(100):
        tiled = rng.random() < 0.7
        B, tw = int(rng.choice([1, 1, 2, 3])), int(rng.integers(0, 2))
        T = int(rng.integers(129, 900)) if tiled else int(rng.integers(1, 300))
        N = int(rng.integers(8, 70)) * 8 if tiled else int(rng.integers(1, 300))
        K = int(rng.integers(1, 12)) * 64 if tiled else int(rng.integers(0, 300))
        if tiled and tw and rng.random() < 0.5:
            N = int(rng.integers(64, 500))
        al = 8 if tiled else 1
        ldx, ldy = K + int(rng.integers(0, 4)) * al, N + int(rng.integers(0, 9))
        wr, wc = (N, K) if tw else (K, N)
        ldw = wc + int(rng.integers(0, 4)) * al
        sx, sw, sy = T * ldx + int(rng.integers(0, 3)) * al, wr * ldw + int(rng.integers(0, 3)) * al, T * ldy + int(rng.integers(0, 5))
        x, w = rng.standard_normal(B * sx + 8).astype(np.float16), (rng.standard_normal(B * sw + 8) * 0.5).astype(np.float16)
        y0 = rng.standard_normal(B * sy).astype(np.float32)
        acc = bool(rng.integers(0, 2))
        yb = DevBuf.of(g, y0)
        ops.gemm_batch_h(B, tw, T, N, K, DevBuf.of(g, x), ldx, sx, DevBuf.of(g, w), ldw, sw, yb, ldy, sy, acc)
        got = yb.read(np.float32)
        written = np.zeros(B * sy, bool)
        what = "product %d: batch %d, w%s, %d x %d x %d, rows %d / %d / %d apart, adding %d" % (it, B, "^T" if tw else "", T, N, K, ldx, ldw, ldy, acc)
        for b in range(B):
            xm = x[b * sx:b * sx + T * ldx].reshape(T, ldx)[:, :K]
            wm = w[b * sw:b * sw + wr * ldw].reshape(wr, ldw)[:, :wc]
            wt = wm.T if tw else wm
            ym = got[b * sy:b * sy + T * ldy].reshape(T, ldy)[:, :N]
            ref = xm.astype(np.float64) @ wt.astype(np.float64) + (y0[b * sy:b * sy + T * ldy].reshape(T, ldy)[:, :N] if acc else 0.0)
            assert (np.abs(ym - ref) <= _bound(xm, wt, K) + 2.0 ** -23 * np.abs(ref)).all(), what
            written[b * sy:b * sy + T * ldy].reshape(T, ldy)[:, :N] = True
        assert np.array_equal(got[~written], y0[~written]), what


@pytest.mark.parametrize("T,H,pos0,K", [(40, 64, 3000, 16), (33, 16, 500, 8), (70, 128, 12000, 64)])
def test_glm_prompt_chain_call_for_call(ops, T, H, pos0, K):
    """GLM's prompt branch as its engine calls the library (llm/glm5next/src/engine.rs:1906-1940): each row's cells as a list,
    the cells gathered out of the half cache 32 rows at a time, queries to half, a batch of products a row's heads against
    its own cells, the masked softmax, the weights to half, the batch of weighted sums - against ns_mla_attend_sel over
    the same lists."""
    g = ops.gpu
    lat, scale = 512, 1.0 / np.sqrt(192.0)
    n = pos0 + T
    rng = np.random.default_rng(T + K)
    cache = _half(41 + T, (n, lat), 0.6)
    qa = orc.randn(42 + T, (T * H, lat)).astype(np.float32)
    sel = np.stack([np.sort(rng.choice((pos0 + t + 1) // 4, K, replace=False)) for t in range(T)]).astype(np.int32)
    cnt = np.full(T, K, np.int32)
    cnt[::7] = -1 if pos0 + T <= 2560 else K // 2               # dense rows where the pass allows them, shorter lists else
    cd, qd, seld, cntd = DevBuf.of(g, cache), DevBuf.of(g, qa), DevBuf.of(g, sel), DevBuf.of(g, cnt)
    fused = DevBuf(g, T * H * lat * 4)
    ops.mla_attend(qd, cd, fused, T, H, lat, pos0, scale, sel=seld, sel_cnt=cntd, K=K)
    want = fused.read(np.float32).reshape(T * H, lat)
    dense = bool((cnt < 0).any())
    nc = ((pos0 + T if dense else 4 * K + 3) + 63) // 64 * 64
    idx, cb = DevBuf(g, T * nc * 4), DevBuf(g, T * 4)
    ops.mla_cells(T, K, pos0, idx, cb, nc, seld, cntd)
    RB = 32
    gh, qh = DevBuf(g, RB * nc * lat * 2), DevBuf(g, RB * H * lat * 2)
    sb, ph = DevBuf(g, RB * H * nc * 4), DevBuf(g, RB * H * nc * 2)
    u = DevBuf(g, T * H * lat * 4)
    u.fill(0xFF)
    for r0 in range(0, T, RB):
        tr = min(RB, T - r0)
        ops.gather_h(cd, n, idx.view(r0 * nc * 4, tr * nc * 4), gh, tr * nc, lat)
        ops.to_f16(qd.view(r0 * H * lat * 4, tr * H * lat * 4), qh, tr * H * lat)
        ops.gemm_batch_h(tr, True, H, nc, lat, qh, lat, H * lat, gh, lat, nc * lat, sb, nc, H * nc)
        ops.softmax_masked(sb, tr, H, nc, cb.view(r0 * 4, tr * 4), scale)
        ops.to_f16(sb, ph, tr * H * nc)
        ops.gemm_batch_h(tr, False, H, lat, nc, ph, nc, H * nc, gh, lat, nc * lat, u.view(r0 * H * lat * 4, tr * H * lat * 4), lat, H * lat)
    chain = u.read(np.float32).reshape(T * H, lat)
    assert np.abs(chain - want).max() <= 2e-3
    assert np.linalg.norm(chain - want) <= 1e-3 * np.linalg.norm(want)


def test_gather_h_rows(ops):
    g = ops.gpu
    rows, C, n = 5000, 512, 3333
    src = np.arange(rows * C, dtype=np.uint32).astype(np.uint16).reshape(rows, C)
    idx = np.random.default_rng(9).integers(0, rows, n).astype(np.int32)
    out = DevBuf(g, n * C * 2 + 64)
    out.fill(0xEE)
    ops.gather_h(DevBuf.of(g, src), rows, DevBuf.of(g, idx), out, n, C)
    got = out.read(np.uint16)
    assert np.array_equal(got[:n * C].reshape(n, C), src[idx]) and (got[n * C:] == 0xEEEE).all()
    with pytest.raises(Error, match="multiple of 8"):
        ops.gather_h(DevBuf.of(g, src), rows, DevBuf.of(g, idx), out, 4, 100)
