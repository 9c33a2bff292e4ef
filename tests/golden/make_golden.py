#!/usr/bin/env python3
"""Writes the golden fixtures of the attention path: inputs, expected cache bytes and expected float64 results, each from
the DEFINITION evaluated in numpy here - not from the oracle and not from the GPU library - so that an edit to either
cannot move the bar unnoticed.

    python tests/golden/make_golden.py        (rewrites tests/golden/*.npz and MANIFEST.sha256)

Rules restated (their sources are the public formats the reference follows):
  half / bfloat16 rows   IEEE round to nearest even (numpy.float16; bfloat16 by the add-0x7FFF-plus-lsb rule)
  q8_0 rows              ggml quantize_row_q8_0_ref on blocks of 32: d = amax / 127, q = round-half-away(x / d), the int8
                         values of a row first, then its half scales (kernels/llm/qwen35/q35.cpp:281-326)
  q4_0 rows              ggml quantize_row_q4_0_ref: d = (value of largest magnitude) / -8, q = min(15, trunc(x / d + 8.5)),
                         byte j of a block = value j | value j + 16 << 4; nibbles first, then the half scales
  GLM q8 latent rows     [16 half scales][512 int8]: the scale amax / 127 rounded to half BEFORE it divides, round half
                         away from zero, clamp to +-127 (kernels/llm/glm5next/glm.cpp:1282-1299)
  attention              softmax(q K^T scale + causal / window mask) V over the widened cache, float64
  absorbed MLA           softmax(qa C^T scale) C[:, :512] over the half latent cache, float64
  YaRN rope              ggml's rope_yarn on adjacent pairs: the angle pos * base^(-i0 / n) scaled by freq_scale, mixed
                         with the unscaled one by the ramp between the correction dims times ext_factor; cos and sin
                         times mscale (kernels/llm/deepseek2/ds2.cpp:15-34, 59-83), float64
  GLM's indexer          pooled key = the softmax over a pool's 4 members of (gate + ape) applied to their keys; pool score =
                         sum over heads of max(S, 0) w, -inf for pools a row does not see; the K best as ascending
                         positions, ties at the K-th value to the lowest positions (kernels/llm/glm5next/glm.cpp:876-1019)
The files are loaded with numpy.load(allow_pickle=False). A file whose arrays would not change is left as it is (a zip's
bytes carry its writing time)."""
import hashlib
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def f2bf(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf2f(b):
    return (b.astype(np.uint32) << 16).view(np.float32)


def q8_0(x):
    x = x.reshape(-1, 32).astype(np.float32)
    d = (np.abs(x).max(axis=1) / np.float32(127.0)).astype(np.float32)
    idv = np.where(d != 0, np.float32(1.0) / np.where(d != 0, d, 1), 0).astype(np.float32)
    p = (x * idv[:, None]).astype(np.float32)
    return (np.sign(p) * np.floor(np.abs(p) + np.float32(0.5))).astype(np.int8), d.astype(np.float16)


def q4_0(x):
    x = x.reshape(-1, 32).astype(np.float32)
    m = x[np.arange(len(x)), np.abs(x).argmax(axis=1)]
    d = (m / np.float32(-8.0)).astype(np.float32)
    idv = np.where(d != 0, np.float32(1.0) / np.where(d != 0, d, 1), 0).astype(np.float32)
    qv = np.minimum(15, ((x * idv[:, None]).astype(np.float32) + np.float32(8.5)).astype(np.float32).astype(np.int32))
    return (qv[:, :16] | (qv[:, 16:] << 4)).astype(np.uint8), d.astype(np.float16)


def cache_rows(kt, x, Hkv, D):
    """x float32 [T][Hkv * D] -> (bytes [Hkv][T][row bytes], widened values float32 [Hkv][T][D])."""
    T = x.shape[0]
    xh = x.reshape(T, Hkv, D).transpose(1, 0, 2)
    if kt == 0:
        h = xh.astype(np.float16)
        return np.ascontiguousarray(h).view(np.uint8).reshape(Hkv, T, 2 * D), h.astype(np.float32)
    if kt == 3:
        b = f2bf(np.ascontiguousarray(xh))
        return np.ascontiguousarray(b).view(np.uint8).reshape(Hkv, T, 2 * D), bf2f(b)
    if kt == 1:
        q, d = q8_0(np.ascontiguousarray(xh))
        rows = np.concatenate([q.reshape(Hkv, T, D).view(np.uint8), np.ascontiguousarray(d.reshape(Hkv, T, D // 32)).view(np.uint8).reshape(Hkv, T, D // 16)], axis=2)
        return rows, (q.astype(np.float32) * d.astype(np.float32)[:, None]).reshape(Hkv, T, D)
    by, d = q4_0(np.ascontiguousarray(xh))
    rows = np.concatenate([by.reshape(Hkv, T, D // 2), np.ascontiguousarray(d.reshape(Hkv, T, D // 32)).view(np.uint8).reshape(Hkv, T, D // 16)], axis=2)
    nib = np.concatenate([by & 15, by >> 4], axis=1).astype(np.float32) - 8
    return rows, (nib * d.astype(np.float32)[:, None]).reshape(Hkv, T, D)


def attention(q, K, V, Hq, Hkv, D, p0, win, causal=True):
    T, G, s = q.shape[0], Hq // Hkv, 1.0 / np.sqrt(D)
    out = np.zeros((T, Hq, D))
    for r in range(T):
        pos = p0 + r
        end = pos + 1 if causal else p0 + T
        first = max(0, pos + 1 - win) if win > 0 else 0
        for h in range(Hq):
            k, v = K[h // G, first:end].astype(np.float64), V[h // G, first:end].astype(np.float64)
            sc = k @ q[r, h * D:(h + 1) * D].astype(np.float64) * s
            e = np.exp(sc - sc.max())
            out[r, h] = (e / e.sum()) @ v
    return out.reshape(T, Hq * D)


def glm_q8rows(x):
    n, L = x.shape
    b = x.reshape(n, L // 32, 32).astype(np.float32)
    d = (np.abs(b).max(axis=2) / np.float32(127.0)).astype(np.float32).astype(np.float16)
    df = d.astype(np.float32)
    inv = np.where(df > 0, np.float32(1.0) / np.where(df > 0, df, 1), 0).astype(np.float32)
    p = (b * inv[:, :, None]).astype(np.float32)
    q = np.clip(np.sign(p) * np.floor(np.abs(p) + np.float32(0.5)), -127, 127).astype(np.int8)
    return np.concatenate([np.ascontiguousarray(d).view(np.uint8).reshape(n, L // 16), q.reshape(n, L).view(np.uint8)], axis=1)


def main():
    rng = np.random.default_rng(20240611)
    files = {}
    # ---- GQA attention over every cache form: decode rows, a verify pass, a short prompt with a window
    att = {}
    cases = [("decode", 1, 8, 2, 128, 70, 0), ("verify", 4, 8, 2, 128, 129, 0), ("window", 3, 4, 1, 128, 100, 48), ("prompt", 40, 4, 2, 128, 25, 0),
             ("wide", 2, 6, 1, 256, 40, 0)]
    for name, T, Hq, Hkv, D, p0, win in cases:
        cap = p0 + T
        k = rng.standard_normal((cap, Hkv * D), dtype=np.float32)
        v = rng.standard_normal((cap, Hkv * D), dtype=np.float32)
        q = rng.standard_normal((T, Hq * D), dtype=np.float32).astype(np.float16).astype(np.float32)      # exact in half
        att[name + "_shape"] = np.array([T, Hq, Hkv, D, p0, win], np.int64)
        att[name + "_k"], att[name + "_v"], att[name + "_q"] = k, v, q
        for kt in (0, 1, 2, 3):
            kc, K = cache_rows(kt, k, Hkv, D)
            vc, V = cache_rows(kt, v, Hkv, D)
            qq = q if kt != 3 else bf2f(f2bf(q))
            att["%s_kc%d" % (name, kt)], att["%s_vc%d" % (name, kt)] = kc, vc
            att["%s_out%d" % (name, kt)] = attention(qq, K, V, Hq, Hkv, D, p0, win)
    files["attention.npz"] = att
    # ---- absorbed MLA over a half latent cache [n][512 + 64], and GLM's latent-only form over q8 rows
    T, H, pos0 = 2, 16, 90
    n = pos0 + T
    cache = (rng.standard_normal((n, 576), dtype=np.float32) * np.float32(0.5)).astype(np.float16)
    qa = rng.standard_normal((T, H, 576), dtype=np.float32).astype(np.float16).astype(np.float32)
    scale = 1.0 / np.sqrt(192.0)
    c = cache.astype(np.float64)
    u = np.zeros((T, H, 512))
    for t in range(T):
        for h in range(H):
            s = c[:pos0 + t + 1] @ qa[t, h].astype(np.float64) * scale
            e = np.exp(s - s.max())
            u[t, h] = (e / e.sum()) @ c[:pos0 + t + 1, :512]
    x = rng.standard_normal((n, 512), dtype=np.float32) * np.float32(0.5)
    x[3, 32:64] = 0.0                                                                    # a zero block
    x[4, 0] = 70000.0                                                                    # a scale past half's range
    rows = glm_q8rows(x)
    files["mla.npz"] = {"shape": np.array([T, H, pos0], np.int64), "cache": cache.view(np.uint16), "qa": qa, "scale": np.array([scale]), "u": u,
                        "glm_x": x, "glm_rows": rows}
    # ---- the steps either side of the latent attention: YaRN rope on a decode step's q_pe, GLM's indexer
    r2 = np.random.default_rng(20240612)
    T, H, head, off, n_dims, pos0 = 3, 4, 192, 128, 64, 1000
    xr = r2.standard_normal((T, H * head), dtype=np.float32)
    yarn = np.array([10000.0, 0.025, 1.0, 1.3, 10.0, 23.0])             # base, freq_scale, ext_factor, mscale, corr dims
    i = np.arange(n_dims // 2)
    ramp = 1.0 - np.clip((i - yarn[4]) / max(0.001, yarn[5] - yarn[4]), 0.0, 1.0)
    yr = xr.astype(np.float64)
    for t in range(T):
        extrap = (pos0 + t) * yarn[0] ** (-2.0 * i / n_dims)
        theta = yarn[1] * extrap * (1 - ramp * yarn[2]) + extrap * ramp * yarn[2]
        c, sn = np.cos(theta) * yarn[3], np.sin(theta) * yarn[3]
        for h in range(H):
            a = xr[t, h * head + off:h * head + off + n_dims].astype(np.float64)
            yr[t, h * head + off:h * head + off + n_dims:2] = a[0::2] * c - a[1::2] * sn
            yr[t, h * head + off + 1:h * head + off + n_dims:2] = a[0::2] * sn + a[1::2] * c
    D, n_tok, hh, K = 32, 50, 4, 5
    ik, ig = r2.standard_normal((n_tok, D), dtype=np.float32), r2.standard_normal((n_tok, D), dtype=np.float32)
    ape = r2.standard_normal((4, D), dtype=np.float32) * np.float32(0.5)
    pooled = np.zeros((n_tok // 4, D))
    for j in range(n_tok // 4):
        lg = ig[4 * j:4 * j + 4].astype(np.float64) + ape
        wgt = np.exp(lg - lg.max(axis=0))
        pooled[j] = (wgt * ik[4 * j:4 * j + 4]).sum(axis=0) / wgt.sum(axis=0)
    Tq, q0 = 3, n_tok - 3                                                 # a verify pass of 3 rows at positions 47..49
    npool = n_tok // 4
    S = r2.standard_normal((Tq * hh, npool), dtype=np.float32)
    S[:, 5] = S[:, 3]                                                     # equal scores: the tie rule decides
    w = np.abs(r2.standard_normal((Tq, hh), dtype=np.float32))
    score = np.full((Tq, npool), -np.inf)
    for r in range(Tq):
        nv = (q0 + r + 1) // 4
        score[r, :nv] = (np.maximum(S[r * hh:(r + 1) * hh, :nv].astype(np.float64), 0.0) * w[r].astype(np.float64)[:, None]).sum(axis=0)
    score32 = score.astype(np.float32)
    score32[:, 5] = score32[:, 3]
    sel = np.stack([np.sort(np.lexsort((np.arange(npool), -score32[r].astype(np.float64)))[:K]) for r in range(Tq)]).astype(np.int32)
    files["select.npz"] = {"rope_shape": np.array([T, H, head, off, n_dims, pos0], np.int64), "rope_x": xr, "rope_yarn": yarn, "rope_y": yr,
                           "idx_shape": np.array([D, n_tok, hh, K, Tq, q0], np.int64), "idx_ik": ik, "idx_ig": ig, "idx_ape": ape,
                           "idx_pooled": pooled, "idx_S": S, "idx_w": w, "idx_score": score, "idx_score32": score32, "idx_sel": sel}
    lines = []
    for fn, arrs in files.items():
        path = os.path.join(HERE, fn)
        same = False
        if os.path.exists(path):
            with np.load(path, allow_pickle=False) as old:
                same = set(old.files) == set(arrs) and all(np.array_equal(old[k], arrs[k], equal_nan=True) and old[k].dtype == np.asarray(arrs[k]).dtype for k in arrs)
        if not same:
            np.savez_compressed(path, **arrs)
        lines.append("%s  %s" % (hashlib.sha256(open(path, "rb").read()).hexdigest(), fn))
    open(os.path.join(HERE, "MANIFEST.sha256"), "w").write("\n".join(lines) + "\n")
    print("\n".join(lines))


if __name__ == "__main__":
    main()
