"""ctypes binding of the CPU oracle (oracle.c -> liboracle.so). TEST INFRASTRUCTURE: imported only by tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg; the product (nextsycl_amd) never imports it."""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "liboracle.so")


def build(force=False):
    """Compile oracle.c with gcc (the recipe is oracle/Makefile)."""
    if force or not os.path.exists(LIB) or os.path.getmtime(LIB) < os.path.getmtime(os.path.join(HERE, "oracle.c")):
        subprocess.run(["make", "-C", HERE, "-B", "liboracle.so"], check=True, capture_output=True)
    return LIB


_lib = None
i64, f32, f64, u64 = C.c_int64, C.c_float, C.c_double, C.c_uint64
P = C.c_void_p


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        L = C.CDLL(LIB)
        sig = {
            "orc_f2h": (C.c_uint16, [f32]), "orc_h2f": (f32, [C.c_uint16]), "orc_f2bf": (C.c_uint16, [f32]), "orc_bf2f": (f32, [C.c_uint16]),
            "orc_f2h_n": (None, [P, P, i64]), "orc_h2f_n": (None, [P, P, i64]), "orc_f2bf_n": (None, [P, P, i64]), "orc_bf2f_n": (None, [P, P, i64]),
            "orc_uniform_f32": (None, [u64, P, i64]), "orc_randn_f32": (None, [u64, f64, P, i64]),
            "orc_kv_row_bytes": (i64, [C.c_int, i64]),
            "orc_kv_dequant": (None, [P, C.c_int, i64, i64, i64, P]),
            "orc_kv_store": (C.c_int, [C.c_int, P, i64, P, i64, i64, i64, i64, i64, i64, C.c_int, P, P]),
            "orc_kv_store_q": (C.c_int, [C.c_int, P, i64, P, i64, i64, i64, i64, i64, i64, P, P]),
            "orc_fwht32": (None, [P, i64, i64, i64]),
            "orc_glm_to_q8row": (None, [P, P, i64, i64]),
            "orc_q35_split_keys": (i64, [i64, i64, i64]), "orc_q35_splits": (i64, [i64, i64, i64]),
            "orc_mg_split_keys": (i64, [i64, i64, i64]), "orc_mg_splits": (i64, [i64, i64, i64]), "orc_mg_seen": (i64, [i64, i64, i64, C.c_int]),
            "orc_dec_split": (i64, [i64, i64]), "orc_dec_splits": (i64, [i64, i64]),
            "orc_q35_attn_decode_scratch": (i64, [i64, i64, i64, i64, i64]),
            "orc_attn_exact": (C.c_int, [P, i64, P, P, C.c_int, C.c_int, i64, i64, i64, i64, i64, i64, i64, C.c_int, i64, C.c_int, P]),
            "orc_attn_f64": (C.c_int, [P, i64, P, P, C.c_int, C.c_int, i64, i64, i64, i64, i64, i64, i64, C.c_int, f64, P]),
            "orc_attn_f64_block": (C.c_int, [P, i64, P, P, C.c_int, C.c_int, i64, i64, i64, i64, i64, i64, i64, f64, P]),
            "orc_attn_probs": (C.c_int, [C.c_int, P, P, i64, i64, i64, i64, i64, C.c_int, P]),
            "orc_glm_mla_attend_f32": (None, [P, P, P, i64, i64, i64, i64, f32]),
            "orc_glm_gather_q8_h": (None, [P, P, P, i64, i64]),
            "orc_glm_mla_cells": (None, [P, P, i64, i64, i64, P, P, i64]),
            "orc_glm_softmax_masked": (None, [P, i64, i64, i64, P, f32]),
            "orc_attn_flash_model": (C.c_int, [P, i64, P, P, C.c_int, C.c_int, i64, i64, i64, i64, i64, i64, i64, i64, P]),
            "orc_mm3_attend": (C.c_int, [P, P, P, P, i64, i64, i64, i64, f32]),
            "orc_mm3_attend_sel": (C.c_int, [P, P, P, P, i64, P, i64, i64, i64, i64, f32]),
            "orc_mm3_idx_scores": (None, [P, P, P, i64, i64, i64, i64, i64]),
            "orc_mm3_idx_topk": (None, [P, P, i64, i64, i64, i64]),
            "orc_glm_mla_attend_sel": (None, [P, P, C.c_int, P, i64, i64, i64, i64, f32, P, P, i64]),
            "orc_ds2_kv_store": (C.c_int, [P, P, f32, P, i64, i64, i64, i64, f32, f32, f32, f32, f32, f32]),
            "orc_idx_pool": (None, [P, P, P, P, P, i64, i64, i64]),
            "orc_idx_score": (None, [P, P, P, i64, i64, i64, i64, i64, i64]),
            "orc_topk": (None, [P, P, i64, i64, i64, i64]),
            "orc_ds2_rope": (C.c_int, [P, i64, i64, i64, i64, i64, i64, i64, f32, f32, f32, f32, f32, f32, P, i64, i64]),
            "orc_mla_absorb": (None, [P, P, P, i64, i64, i64, i64, i64]),
            "orc_mla_decode_u": (None, [P, P, P, i64, i64, i64, i64, i64, f32]),
            "orc_mla_vb": (None, [P, P, P, i64, i64, i64, i64]),
            "orc_q6k_row512": (None, [P, P]),
            "orc_mla_absorb_q6k": (None, [P, P, P, i64, i64]),
            "orc_mla_vb_q6k": (None, [P, P, P, i64, i64]),
            "orc_mla_f64": (None, [P, P, P, i64, i64, i64, i64, i64, f64]),
            "orc_glm_mla_attend": (None, [P, P, C.c_int, P, i64, i64, i64, i64, f32]),
            "orc_q35_norm_rope": (C.c_int, [P, i64, i64, P, i64, i64, i64, i64, P, f32, i64, f32, i64, P, i64, i64, i64]),
            "orc_mg_norm_rope": (C.c_int, [P, i64, P, i64, i64, i64, i64, P, f32, C.c_int, f32, i64]),
            "orc_mm3_norm_rope_row": (C.c_int, [P, P, P, C.c_int, i64, i64, i64, f32, f32]),
            "orc_compare": (None, [P, P, i64, P, P, P]),
            "orc_threads": (C.c_int, []),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(P)


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


# ---- conversions -------------------------------------------------------------------------------------------------
def f2h(x):
    x = _c(x, np.float32)
    y = np.empty(x.shape, np.uint16)
    lib().orc_f2h_n(_p(x), _p(y), x.size)
    return y


def h2f(x):
    x = _c(x, np.uint16)
    y = np.empty(x.shape, np.float32)
    lib().orc_h2f_n(_p(x), _p(y), x.size)
    return y


def f2bf(x):
    x = _c(x, np.float32)
    y = np.empty(x.shape, np.uint16)
    lib().orc_f2bf_n(_p(x), _p(y), x.size)
    return y


def bf2f(x):
    x = _c(x, np.uint16)
    y = np.empty(x.shape, np.float32)
    lib().orc_bf2f_n(_p(x), _p(y), x.size)
    return y


# ---- seeded inputs -----------------------------------------------------------------------------------------------
def uniform(seed, n):
    y = np.empty(n, np.float32)
    lib().orc_uniform_f32(seed, _p(y), n)
    return y


def randn(seed, shape, sigma=1.0):
    n = int(np.prod(shape))
    y = np.empty(n, np.float32)
    lib().orc_randn_f32(seed, float(sigma), _p(y), n)
    return y.reshape(shape)


def randn_f16(seed, shape, sigma=1.0):
    """N(0, sigma) rounded to half: (bits uint16, the rounded values as float32)."""
    b = f2h(randn(seed, shape, sigma))
    return b, h2f(b)


def randn_bf16(seed, shape, sigma=1.0):
    b = f2bf(randn(seed, shape, sigma))
    return b, bf2f(b)


# ---- cache rows --------------------------------------------------------------------------------------------------
def kv_row_bytes(kt, D):
    return lib().orc_kv_row_bytes(kt, D)


def kv_store(kt, k, v, Hkv, D, cap, p0, kc=None, vc=None, ring=False):
    """k, v float32 [T][Hkv*D] -> caches (uint8 [Hkv][cap][row bytes]); kt 0 half, 3 bfloat16, 1 q8_0, 2 q4_0."""
    k, v = _c(k, np.float32), _c(v, np.float32)
    T = k.shape[0]
    rb = kv_row_bytes(kt, D)
    if kc is None:
        kc = np.zeros((Hkv, cap, rb), np.uint8)
        vc = np.zeros((Hkv, cap, rb), np.uint8)
    if kt in (0, 3):
        rc = lib().orc_kv_store(kt, _p(k), k.shape[1], _p(v), v.shape[1], T, Hkv, D, cap, p0, int(ring), _p(kc), _p(vc))
    else:
        rc = lib().orc_kv_store_q(kt, _p(k), k.shape[1], _p(v), v.shape[1], T, Hkv, D, cap, p0, _p(kc), _p(vc))
    if rc:
        raise ValueError("orc_kv_store: bad arguments")
    return kc, vc


def kv_dequant(rows, kt, D):
    rows = _c(rows, np.uint8)
    rb = kv_row_bytes(kt, D)
    n = rows.size // rb
    out = np.empty((n, D), np.float32)
    lib().orc_kv_dequant(_p(rows), kt, D, n, rb, _p(out))
    return out.reshape(rows.shape[:-1] + (D,))


def fwht32(x):
    x = _c(x, np.float32).copy()
    rows, n = x.reshape(-1, x.shape[-1]).shape
    lib().orc_fwht32(_p(x), rows, n, n)
    return x


def glm_to_q8row(x, L):
    x = _c(x, np.float32)
    n = x.size // L
    y = np.zeros((n, L // 32 * 2 + L), np.uint8)
    lib().orc_glm_to_q8row(_p(x), _p(y), n, L)
    return y


# ---- attention ---------------------------------------------------------------------------------------------------
def attn_exact(q, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=0, causal=True, pm=False, groups=None, split_single_only=False):
    q = _c(q, np.float32).reshape(T, Hq * D)
    out = np.empty((T, Hq * D), np.float32)
    g = groups if groups is not None else max(1, Hq // 4)
    rc = lib().orc_attn_exact(_p(q), Hq * D, _p(kc), _p(vc), kt, int(pm), T, Hq, Hkv, D, cap, p0, win, int(causal), g, int(split_single_only), _p(out))
    if rc:
        raise ValueError("orc_attn_exact: bad arguments")
    return out


def attn_f64(q, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=0, causal=True, pm=False, scale=0.0):
    q = _c(q, np.float32).reshape(T, Hq * D)
    out = np.empty((T, Hq * D), np.float64)
    rc = lib().orc_attn_f64(_p(q), Hq * D, _p(kc), _p(vc), kt, int(pm), T, Hq, Hkv, D, cap, p0, win, int(causal), float(scale), _p(out))
    if rc:
        raise ValueError("orc_attn_f64: bad arguments")
    return out


def attn_f64_block(q, kc, vc, kt, T, Hq, Hkv, D, cap, p0, kfirst, pm=False, scale=0.0):
    """A draft block: every row sees keys kfirst .. p0 + T - 1 (not causal)."""
    q = _c(q, np.float32).reshape(T, Hq * D)
    out = np.empty((T, Hq * D), np.float64)
    rc = lib().orc_attn_f64_block(_p(q), Hq * D, _p(kc), _p(vc), kt, int(pm), T, Hq, Hkv, D, cap, p0, kfirst, float(scale), _p(out))
    if rc:
        raise ValueError("orc_attn_f64_block: bad arguments")
    return out


def attn_probs(kt, q, kc, Hq, Hkv, D, cap, n, mode, out=None):
    """out [n] += the heads' weights of each key: their mean (mode 0) or largest (1) - ns_q35_attn_probs."""
    q = _c(q, np.float32)
    out = np.zeros(n, np.float32) if out is None else _c(out, np.float32).copy()
    rc = lib().orc_attn_probs(kt, _p(q), _p(kc), Hq, Hkv, D, cap, n, mode, _p(out))
    if rc:
        raise ValueError("orc_attn_probs: bad arguments")
    return out


def attn_flash_model(q, kc, vc, kt, T, Hq, Hkv, D, cap, p0, win=0, kbs=0, pm=False):
    q = _c(q, np.float32).reshape(T, Hq * D)
    out = np.empty((T, Hq * D), np.float32)
    rc = lib().orc_attn_flash_model(_p(q), Hq * D, _p(kc), _p(vc), kt, int(pm), T, Hq, Hkv, D, cap, p0, win, kbs, _p(out))
    if rc:
        raise ValueError("orc_attn_flash_model: bad arguments")
    return out


def mm3_attend(q, kc, vc, T, H, G, pos0, scale, sel=None, K=0):
    q = _c(q, np.float32)
    out = np.empty((T, H * 128), np.float32)
    sp = _p(_c(sel, np.int32)) if sel is not None else None
    rc = lib().orc_mm3_attend_sel(_p(q), _p(kc), _p(vc), sp, K, _p(out), T, H, G, pos0, float(scale))
    if rc:
        raise ValueError("orc_mm3_attend: bad arguments")
    return out


def mm3_idx_scores(iq, ik, T, G, nblk, pos0, local):
    iq, ik = _c(iq, np.float32), _c(ik, np.uint16)
    bs = np.empty((T, G, nblk), np.float32)
    lib().orc_mm3_idx_scores(_p(iq), _p(ik), _p(bs), T, G, nblk, pos0, local)
    return bs


def mm3_idx_topk(bs, K):
    """(sel [T][G][K], the scores as the selection leaves them)."""
    bs = np.array(bs, np.float32)
    T, G, nblk = bs.shape
    sel = np.empty((T, G, K), np.int32)
    lib().orc_mm3_idx_topk(_p(bs), _p(sel), T, G, nblk, K)
    return sel, bs


# ---- MLA ---------------------------------------------------------------------------------------------------------
def ds2_kv_store(kv, w, eps, cache, T, L, R, pos0, freq_base, freq_scale, ext_factor, mscale, corr0, corr1):
    kv, w = _c(kv, np.float32), _c(w, np.float32)
    rc = lib().orc_ds2_kv_store(_p(kv), _p(w), eps, _p(cache), T, L, R, pos0, freq_base, freq_scale, ext_factor, mscale, corr0, corr1)
    if rc:
        raise ValueError("orc_ds2_kv_store: bad arguments")
    return cache


def ds2_rope(x, T, H, row, head, off, n_dims, pos0, freq_base, freq_scale, ext_factor, mscale, corr0, corr1, out=None, out_row=0, out_head=0):
    """ns_ds2_rope: x (float32, modified in place and returned); out: an array the rotated part is also written into."""
    x = _c(x, np.float32)
    rc = lib().orc_ds2_rope(_p(x), T, H, row, head, off, n_dims, pos0, freq_base, freq_scale, ext_factor, mscale, corr0, corr1,
                            _p(out) if out is not None else None, out_row, out_head)
    if rc:
        raise ValueError("orc_ds2_rope: bad arguments")
    return x


def glm_idx_pool(ring, ik, ig, ape, pooled, pos0, T, D):
    """ns_idx_pool: ring [8][2 D] and pooled [pools][D] (float32, contiguous) are updated in place."""
    lib().orc_idx_pool(_p(ring), _p(_c(ik, np.float32)), _p(_c(ig, np.float32)), _p(_c(ape, np.float32)), _p(pooled), pos0, T, D)


def glm_idx_score(S, w, score, T, H, j0, n, pos0):
    """ns_idx_score: score [T][ld] (float32, contiguous) gets columns j0 .. j0 + n - 1."""
    lib().orc_idx_score(_p(_c(S, np.float32)), _p(_c(w, np.float32)), _p(score), T, H, j0, n, score.shape[1], pos0)


def glm_topk(score, n, K):
    """ns_topk over score [T][ld]: sel [T][K] int32 (entries past a row's n stay -1)."""
    score = _c(score, np.float32)
    T, ld = score.shape
    sel = np.full((T, K), -1, np.int32)
    lib().orc_topk(_p(score), _p(sel), T, n, ld, K)
    return sel


def mla_absorb(q, kb, T, H, L=512, R=64, NOPE=128):
    q, kb = _c(q, np.float32), _c(kb, np.uint16)
    qa = np.empty((T, H, L + R), np.float32)
    lib().orc_mla_absorb(_p(q), _p(kb), _p(qa), T, H, L, R, NOPE)
    return qa


def mla_decode_u(qa, cache, T, H, pos0, scale, L=512, R=64):
    qa, cache = _c(qa, np.float32), _c(cache, np.uint16)
    u = np.empty((T, H, L), np.float32)
    lib().orc_mla_decode_u(_p(qa), _p(cache), _p(u), T, H, L, R, pos0, float(scale))
    return u


def mla_vb(u, vb, T, H, L=512, V=128):
    u, vb = _c(u, np.float32), _c(vb, np.uint16)
    out = np.empty((T, H, V), np.float32)
    lib().orc_mla_vb(_p(u), _p(vb), _p(out), T, H, L, V)
    return out


def q6k_rows512(rows):
    """Q6_K rows of 512 values (420 bytes each) widened to float32 [n][512]."""
    rows = _c(rows, np.uint8).reshape(-1, 420)
    out = np.empty((rows.shape[0], 512), np.float32)
    for i in range(rows.shape[0]):
        lib().orc_q6k_row512(_p(rows[i]), _p(out[i]))
    return out


def mla_absorb_q6k(q, kvb, T, H):
    q, kvb = _c(q, np.float32), _c(kvb, np.uint8)
    qa = np.empty((T, H, 576), np.float32)
    lib().orc_mla_absorb_q6k(_p(q), _p(kvb), _p(qa), T, H)
    return qa


def mla_vb_q6k(u, kvb, T, H):
    u, kvb = _c(u, np.float32), _c(kvb, np.uint8)
    out = np.empty((T, H, 128), np.float32)
    lib().orc_mla_vb_q6k(_p(u), _p(kvb), _p(out), T, H)
    return out


def mla_f64(qa, cache, T, H, pos0, scale, L=512, R=64):
    qa, cache = _c(qa, np.float32), _c(cache, np.uint16)
    u = np.empty((T, H, L), np.float64)
    lib().orc_mla_f64(_p(qa), _p(cache), _p(u), T, H, L, R, pos0, float(scale))
    return u


def glm_mla_attend_sel(qa, cache, q8, T, H, L, pos0, scale, sel, sel_cnt, K):
    qa = _c(qa, np.float32)
    u = np.empty((T, H * L), np.float32)
    lib().orc_glm_mla_attend_sel(_p(qa), _p(cache), int(q8), _p(u), T, H, L, pos0, float(scale), _p(_c(sel, np.int32)), _p(_c(sel_cnt, np.int32)), K)
    return u


def glm_mla_attend(qa, cache, q8, T, H, L, pos0, scale):
    qa = _c(qa, np.float32)
    cache = np.ascontiguousarray(cache)
    u = np.empty((T, H, L), np.float32)
    lib().orc_glm_mla_attend(_p(qa), _p(cache), int(q8), _p(u), T, H, L, pos0, float(scale))
    return u


def glm_mla_attend_f32(qa, c, T, H, L, pos0, scale):
    """ns_mla_attend: the dense form over a float32 latent cache c [n][L]."""
    qa, c = _c(qa, np.float32), _c(c, np.float32)
    u = np.empty((T, H, L), np.float32)
    lib().orc_glm_mla_attend_f32(_p(qa), _p(c), _p(u), T, H, L, pos0, float(scale))
    return u


def glm_gather_q8_h(src, idx, L):
    """ns_gather_q8_h: the q8 latent rows idx of src widened to half bits [n][L]."""
    src, idx = np.ascontiguousarray(src, np.uint8), _c(idx, np.int32)
    out = np.empty((idx.size, L), np.uint16)
    lib().orc_glm_gather_q8_h(_p(src), _p(idx), _p(out), idx.size, L)
    return out


def glm_mla_cells(T, K, pos0, NC, sel=None, sel_cnt=None):
    """ns_mla_cells: (idx [T][NC] int32, n [T] int32) - each row's cells as a list."""
    idx, n = np.empty((T, NC), np.int32), np.empty(T, np.int32)
    if sel_cnt is not None:
        sel, sel_cnt = _c(sel, np.int32), _c(sel_cnt, np.int32)
    lib().orc_glm_mla_cells(_p(sel) if sel_cnt is not None else None, _p(sel_cnt) if sel_cnt is not None else None, T, K, pos0, _p(idx), _p(n), NC)
    return idx, n


def glm_softmax_masked(S, R, H, NC, n, scale):
    """ns_softmax_masked: the masked row softmax of S [R H][NC] (a copy)."""
    out, n = np.array(S, np.float32, order="C").reshape(R * H, NC), _c(n, np.int32)
    lib().orc_glm_softmax_masked(_p(out), R, H, NC, _p(n), float(scale))
    return out


# ---- comparisons -------------------------------------------------------------------------------------------------
# ---- norm + rotary positions ----------------------------------------------------------------------------------------
def q35_norm_rope(x, T, H, D, w, eps, n_rot, theta, p0, pos3=None, sections=(0, 0, 0)):
    """x [T][H][D] float32 -> RMS norm (w None: none) + rotate-half over the first n_rot (ns_q35_qk_norm_rope / _pos / ns_q35_rope)."""
    x = _c(x, np.float32).reshape(T, H * D)
    y = np.empty_like(x)
    wp = _p(_c(w, np.float32)) if w is not None else None
    pp = _p(_c(pos3, np.int32)) if pos3 is not None else None
    rc = lib().orc_q35_norm_rope(_p(x), H * D, D, _p(y), H * D, T, H, D, wp, eps, n_rot, theta, p0, pp, *sections)
    if rc:
        raise ValueError("orc_q35_norm_rope: bad arguments")
    return y


def mg_norm_rope(x, T, H, D, w, eps, rope, theta, p0):
    x = _c(x, np.float32).reshape(T, H * D)
    y = np.empty_like(x)
    rc = lib().orc_mg_norm_rope(_p(x), H * D, _p(y), H * D, T, H, D, _p(_c(w, np.float32)), eps, rope, theta, p0)
    if rc:
        raise ValueError("orc_mg_norm_rope: bad arguments")
    return y


def mm3_norm_rope_row(row, w, rot, n_rot, pos, base, eps, want_half=False):
    """One head row: (new float32 row, half copy or None) of the MiniMax-M3 norm + rotate-half."""
    row = np.array(row, np.float32)
    half = np.empty(row.size, np.uint16) if want_half else None
    wp = _p(_c(w, np.float32)) if w is not None else None
    rc = lib().orc_mm3_norm_rope_row(_p(row), wp, _p(half) if want_half else None, int(rot), row.size, n_rot, pos, base, eps)
    if rc:
        raise ValueError("orc_mm3_norm_rope_row: bad arguments")
    return row, half


# ---- checkpoints: the engines' host loops over a ring cache's runs, restated in numpy (byte moves only)
def ring_kept(w, pos):
    """llm/museglimmer/src/engine.rs:1358-1361."""
    return max(pos - (w - 1), 0) if w > 0 else 0


def ring_save(cache, heads, cap, row, w, pos):
    """One cache's checkpoint buffer: [heads][kept .. pos)[row] bytes out of a ring [heads][cap][row] (slot = p % cap),
    read as the engine does - runs that end at the ring's last slot (llm/museglimmer/src/engine.rs:1479-1494)."""
    cache = np.ascontiguousarray(cache).view(np.uint8).reshape(-1)
    first = ring_kept(w, pos)
    n = pos - first
    b = np.zeros(heads * n * row, np.uint8)
    for h in range(heads):
        p = first
        while p < pos:
            si = p % cap
            run = min(pos - p, cap - si)
            at = (h * n + p - first) * row
            src = (h * cap + si) * row
            b[at:at + run * row] = cache[src:src + run * row]
            p += run
    return b


def ring_restore(cache, b, heads, cap, row, w, pos):
    """`ring_save`'s buffer written back into a ring in place (llm/museglimmer/src/engine.rs:1509-1523)."""
    cache = cache.view(np.uint8).reshape(-1)
    first = ring_kept(w, pos)
    n = pos - first
    if b.size != heads * n * row:
        raise ValueError("a checkpoint of another shape")
    for h in range(heads):
        p = first
        while p < pos:
            si = p % cap
            run = min(pos - p, cap - si)
            at = (h * n + p - first) * row
            dst = (h * cap + si) * row
            cache[dst:dst + run * row] = b[at:at + run * row]
            p += run


def ring_copy(dst, dcap, src, scap, heads, row, first, to):
    """Positions [first, to) of one ring into another of other capacity, in place (llm/museglimmer/src/engine.rs:1334-1346)."""
    dst = dst.view(np.uint8).reshape(-1)
    src = np.ascontiguousarray(src).view(np.uint8).reshape(-1)
    for h in range(heads):
        p = first
        while p < to:
            si, di = p % scap, p % dcap
            run = min(to - p, scap - si, dcap - di)
            d0, s0 = (h * dcap + di) * row, (h * scap + si) * row
            dst[d0:d0 + run * row] = src[s0:s0 + run * row]
            p += run


def checkpoint_file(magic, pos, bufs):
    """The engines' checkpoint file: magic, u64 position, u64 count, then u64 length + bytes a buffer, little-endian
    (llm/museglimmer/src/engine.rs:230-240)."""
    out = bytearray(magic)
    out += int(pos).to_bytes(8, "little") + len(bufs).to_bytes(8, "little")
    for b in bufs:
        b = np.ascontiguousarray(b).view(np.uint8).reshape(-1)
        out += int(b.size).to_bytes(8, "little") + b.tobytes()
    return bytes(out)


def compare(a, b):
    """(max-abs, relative L2, cosine) of a (float32) against b (float64) - the reference's `kernels` check's measures."""
    a = _c(a, np.float32).ravel()
    b = _c(b, np.float64).ravel()
    assert a.size == b.size
    m, r, c = f64(), f64(), f64()
    lib().orc_compare(_p(a), _p(b), a.size, C.byref(m), C.byref(r), C.byref(c))
    return m.value, r.value, c.value


def threads():
    return lib().orc_threads()
