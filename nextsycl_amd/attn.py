"""The attention ABI (include/ns_attn.h) bound by name, and the size-checked wrappers an engine calls.

`Kernels` is the table of function pointers - the counterpart of an engine's `ffi.rs` (llm/qwen35/src/ffi.rs:42-52,
70-136; llm/museglimmer/src/ffi.rs; llm/deepseek2/src/ffi.rs:36-39): every entry point looked up by name when the table
is built, a missing symbol being a load error. `Ops` is the counterpart of `ops.rs` (llm/deepseek2/src/ops.rs:391-445):
each wrapper checks that its buffers hold what the kernel will touch, then makes the C call and turns -1 into
Error("<what>: <ns_last_error>"). The call order of a pass is the engines': kv_store -> *_scratch -> attention
(llm/museglimmer/src/engine.rs:856-873). Nothing here computes: the HIP library does, or the call fails."""
import ctypes as C

from .core import Error, api
from .sys import P, f32, i32, i64

F32, F16, BF16 = 0, 1, 2                       # q / out element types (NS_F32, NS_F16, NS_BF16)
# ns_attn_tune's knobs
TUNE_DEC_WGS, TUNE_PREFILL_SPLITS, TUNE_PREFILL_WAVES, TUNE_MLA_WGS, TUNE_PRE_HPW, TUNE_PREFILL_BF16, TUNE_SCRATCH_MIB = 0, 1, 2, 3, 4, 5, 6
KV_F16, KV_Q8_0, KV_Q4_0, KV_BF16 = 0, 1, 2, 3   # cache forms
ELT = {F32: 4, F16: 2, BF16: 2}


def kv_row_bytes(kt, D):
    """Bytes of one (head, position) row of a cache of form kt (llm/qwen35/src/engine.rs:54-60)."""
    if kt == KV_Q8_0:
        return D + D // 32 * 2
    if kt == KV_Q4_0:
        return D // 2 + D // 32 * 2
    if kt in (KV_F16, KV_BF16):
        return 2 * D
    raise Error("a cache form 0 (half), 1 (q8_0), 2 (q4_0) or 3 (bfloat16)")


# name -> (restype, argtypes): include/ns_attn.h
ATTN_H = {
    "ns_q35_kv_store": (i32, [P, P, i64, P, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_q35_kv_store_q": (i32, [P, i32, P, i64, P, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_mg_kv_store": (i32, [P, P, P, i64, i64, i64, i64, i64, P, P]),
    "ns_attn_kv_store": (i32, [P, i32, i32, P, i64, P, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_attn_kv_dequant": (i32, [P, i32, P, i64, i64, i64, P]),
    "ns_attn_kv_rows_copy": (i32, [P, P, i64, i64, P, i64, i64, i64, i64, i64, i64]),
    "ns_q35_fwht32": (i32, [P, P, i64, i64, i64]),
    "ns_attn_decode_scratch": (i64, [i64, i64, i64, i64, i64, i64]),
    "ns_attn_decode_t": (i32, [P, i32, i32, i32, P, i64, P, P, i64, i64, i64, i64, i64, i64, i64, f32, P, P]),
    "ns_attn_decode_static": (i32, [P, i32, i32, i32, P, i64, P, P, i64, i64, i64, i64, i64, i64, i64, f32, P]),
    "ns_q35_attn_decode_supported": (i32, [i64, i64, i64, i64]),
    "ns_q35_attn_decode_scratch": (i64, [i64, i64, i64, i64, i64]),
    "ns_q35_attn_decode": (i32, [P, P, i64, P, P, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_q35_attn_decode_kv": (i32, [P, i32, P, i64, P, P, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_mg_attn_decode_supported": (i32, [i64, i64, i64, i64]),
    "ns_mg_attn_decode_scratch": (i64, [i64, i64, i64, i64, i64, i64]),
    "ns_mg_attn_decode": (i32, [P, P, P, P, i64, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_attn_prompt_t": (i32, [P, i32, i32, i32, P, i64, P, P, i64, i64, i64, i64, i64, i64, i64, f32, P]),
    "ns_mg_attn_prompt_supported": (i32, [i64, i64, i64, i64]),
    "ns_mg_attn_prompt": (i32, [P, P, P, P, i64, i64, i64, i64, i64, i64, i64, P]),
    "ns_q35_attn_prompt_supported": (i32, [i64, i64, i64, i64]),
    "ns_q35_attn_prompt": (i32, [P, P, i64, P, P, i64, i64, i64, i64, i64, i64, P]),
    "ns_q35_attn_prompt_kv": (i32, [P, i32, P, i64, P, P, i64, i64, i64, i64, i64, i64, P]),
    "ns_nhs_attn_prompt_supported": (i32, [i64, i64, i64, i64]),
    "ns_nhs_attn_prompt": (i32, [P, P, i64, P, P, i64, i64, i64, i64, i64, i64, P]),
    "ns_nhs_attn_decode_supported": (i32, [i64, i64, i64, i64]),
    "ns_nhs_attn_decode_scratch": (i64, [i64, i64, i64, i64, i64]),
    "ns_nhs_attn_decode": (i32, [P, P, i64, P, P, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_q35_attn_scratch": (i64, [i64, i64, i64, i64, i64]),
    "ns_q35_attn": (i32, [P, P, i64, P, P, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_mg_attn_scratch": (i64, [i64, i64, i64, i64, i64, i64, i32]),
    "ns_mg_attn": (i32, [P, P, P, P, i64, i64, i64, i64, i64, i64, i64, i32, P, P]),
    "ns_mg_attn_block_scratch": (i64, [i64, i64, i64, i64, i64, i64]),
    "ns_mg_attn_block": (i32, [P, P, P, P, i64, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_rc_kv_store": (i32, [P, P, i64, P, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_rc_attn_scratch": (i64, [i64, i64, i64, i64, i64, i64]),
    "ns_rc_attn": (i32, [P, P, i64, P, P, i64, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_q35_graph_begin": (i32, [P, C.POINTER(P)]),
    "ns_q35_graph_end": (i32, [P, P]),
    "ns_q35_graph_launch": (i32, [P, P]),
    "ns_q35_graph_free": (None, [P]),
    "ns_rc_flash_prompt_supported": (i32, [i64, i64, i64, i64]),
    "ns_rc_flash_prompt": (i32, [P, P, P, P, i64, i64, i64, i64, i64, i64, i64, P]),
    "ns_rc_flash_decode_supported": (i32, [i64, i64, i64, i64]),
    "ns_rc_flash_decode_scratch": (i64, [i64, i64, i64, i64, i64, i64]),
    "ns_rc_flash_decode": (i32, [P, P, P, P, i64, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_nh_kv_store": (i32, [P, P, i64, P, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_nh_attn_scratch": (i64, [i64, i64, i64, i64, i64]),
    "ns_nh_attn": (i32, [P, P, i64, P, P, i64, i64, i64, i64, i64, i64, P, P]),
    "ns_q35_attn_probs": (i32, [P, i32, P, P, i64, i64, i64, i64, i64, i32, P, P]),
    "ns_mm3s_attend_supported": (i32, [i64, i64, i64]),
    "ns_mm3s_attend": (i32, [P, P, P, P, P, i64, P, i64, i64, i64, i64, f32]),
    "ns_mm3s_attend_x": (i32, [P, P, P, P, P, i64, P, i64, i64, i64, i64, f32]),
    "ns_mm3s_attend_split": (i32, [P, P, P, P, P, i64, P, i64, i64, i64, i64, f32, i64, P]),
    "ns_mm3s_attend_x_split": (i32, [P, P, P, P, P, i64, P, i64, i64, i64, i64, f32, i64, P]),
    "ns_mm3s_attend_block": (i32, [P, P, P, P, P, i64, i64, i64, i64, i64, i64, P]),
    "ns_llm_minimaxm3_attend": (i32, [P, P, P, P, P, i64, P, i64, i64, i64, i64, f32]),
    "ns_llm_minimaxm3_idx_scores": (i32, [P, P, P, P, i64, i64, i64, i64, i64]),
    "ns_llm_minimaxm3_idx_topk": (i32, [P, P, P, i64, i64, i64, i64]),
    "ns_attn_profile": (i32, [P, i32]),
    "ns_attn_copy_probe": (i32, [P, P, P, C.c_size_t]),
    "ns_attn_profile_last": (i32, [P, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "ns_attn_tune": (i32, [i32, i64]),
}


# include/ns_mla.h
MLA_H = {
    "ns_mla_decode_latent_scratch": (i64, [i64, i64, i64]),
    "ns_mla_decode_latent": (i32, [P, i32, P, P, P, i64, i64, i64, i64, f32, P]),
    "ns_ds2_mla_decode": (i32, [P, P, P, P, P, P, i64, i64, i64, f32]),
    "ns_ds2_mla_decode_q6k": (i32, [P, P, P, P, P, i64, i64, i64, f32]),
    "ns_ds2_kv_store": (i32, [P, P, P, f32, P, i64, i64, i64, i64, f32, f32, f32, f32, f32, f32]),
    "ns_ds2_rope": (i32, [P, P, i64, i64, i64, i64, i64, i64, i64, f32, f32, f32, f32, f32, f32, P, i64, i64]),
    "ns_mla_attend_sel": (i32, [P, P, P, P, i64, i64, i64, i64, f32, P, P, i64]),
    "ns_mla_attend_sel_q8": (i32, [P, P, P, P, i64, i64, i64, i64, f32, P, P, i64]),
    "ns_to_q8row": (i32, [P, P, P, i64, i64]),
    "ns_mla_attend": (i32, [P, P, P, P, i64, i64, i64, i64, f32]),
    "ns_gather_q8_h": (i32, [P, P, P, P, i64, i64]),
    "ns_idx_pool": (i32, [P, P, P, P, P, P, i64, i64, i64]),
    "ns_idx_score": (i32, [P, P, P, P, i64, i64, i64, i64, i64, i64]),
    "ns_topk": (i32, [P, P, P, i64, i64, i64, i64]),
    "ns_mla_cells": (i32, [P, P, P, i64, i64, i64, P, P, i64]),
    "ns_softmax_masked": (i32, [P, P, i64, i64, i64, P, f32]),
    "ns_gemm_f16": (i32, [P, i64, i64, i64, P, i64, P, P, i64, i32]),
    "ns_gemm_batch_h": (i32, [P, i64, i32, i64, i64, i64, P, i64, i64, P, i64, i64, P, i64, i64, i32]),
    "ns_to_f16": (i32, [P, P, P, i64]),
    "ns_gather_h": (i32, [P, P, P, P, i64, i64]),
}


# include/ns_pre.h
PRE_H = {
    "ns_q35_qk_norm_rope": (i32, [P, P, i64, i64, P, i64, i64, i64, i64, P, f32, i64, f32, i64]),
    "ns_q35_qk_norm_rope_pos": (i32, [P, P, i64, i64, P, i64, i64, i64, i64, P, f32, i64, f32, P, i64, i64, i64]),
    "ns_rc_qk_norm_rope": (i32, [P, P, i64, i64, P, i64, i64, i64, i64, P, f32, i32, f32, i64]),
    "ns_q35_rope": (i32, [P, P, i64, i64, P, i64, i64, i64, i64, i64, f32, i64]),
    "ns_mg_qk_norm_rope": (i32, [P, P, i64, P, i64, i64, i64, i64, P, f32, i32, f32, i64]),
    "ns_llm_minimaxm3_rope": (i32, [P, P, i64, i64, i64, i64, i64, i64, f32]),
    "ns_mm3s_attn_post": (i32, [P, P, P, P, P, P, P, P, P, P, P, P, P, i64, i64, i64, i64, i64, i64, f32, f32]),
    "ns_attn_pre_store": (i32, [P, i32, i32, i32, i32, P, i64, i64, P, i64, P, i64, i64, P, i64, P, P, f32, i64, f32, i64, i64, i64, i64, i64, i64,
                                P, P]),
}


class Kernels:
    """Every attention entry point bound by name; a missing symbol fails the load."""

    def __init__(self, a=None):
        self.api = a or api()
        for name, (res, args) in list(ATTN_H.items()) + list(MLA_H.items()) + list(PRE_H.items()):
            setattr(self, name[3:], self.api.symbol(name, res, args))


_k = None


def kernels():
    global _k
    if _k is None:
        _k = Kernels()
    return _k


def _need(buf, nbytes, what):
    if buf is None:
        raise Error("%s: no buffer" % what)
    if buf.len < nbytes:
        raise Error("%s: %d bytes, needs %d" % (what, buf.len, nbytes))


class Ops:
    """Checked wrappers over one GPU: the buffers' sizes against what the kernel reads and writes, then the call."""

    def __init__(self, gpu, k=None):
        self.gpu = gpu
        self.k = k or kernels()

    def raw(self):
        return self.gpu.raw

    def ok(self, rc, what):
        if rc != 0:
            raise Error("%s: %s" % (what, self.k.api.error()))

    # ---- measurement
    def profile(self, on):
        self.ok(self.k.attn_profile(self.raw(), int(on)), "profile")

    def profile_last(self):
        """(main kernel ns, merge kernel ns) of the last attention call made with profiling on; waits for it."""
        a, b = C.c_double(), C.c_double()
        self.ok(self.k.attn_profile_last(self.raw(), C.byref(a), C.byref(b)), "profile_last")
        return a.value, b.value

    def tune(self, knob, value):
        """A tuning knob (TUNE_*) to `value`; 0 restores the library's own choice."""
        self.ok(self.k.attn_tune(knob, value), "tune")

    def copy_probe(self, dst, src, nbytes):
        _need(dst, nbytes, "copy_probe dst")
        _need(src, nbytes, "copy_probe src")
        self.ok(self.k.attn_copy_probe(self.raw(), dst.ptr, src.ptr, nbytes), "copy_probe")

    # ---- caches
    def cache_bytes(self, kt, Hkv, cap, D):
        return Hkv * cap * kv_row_bytes(kt, D)

    def kv_store(self, kt, k, ks, v, vs, T, Hkv, D, cap, p0, kc, vc, ring=False):
        """float32 rows k, v [T][Hkv*D] (strides ks, vs floats) into caches of form kt at positions p0.."""
        if T > 0:
            _need(k, ((T - 1) * ks + Hkv * D) * 4, "kv_store k")
            _need(v, ((T - 1) * vs + Hkv * D) * 4, "kv_store v")
        _need(kc, self.cache_bytes(kt, Hkv, cap, D), "kv_store key cache")
        _need(vc, self.cache_bytes(kt, Hkv, cap, D), "kv_store value cache")
        self.ok(self.k.attn_kv_store(self.raw(), kt, int(ring), k.ptr, ks, v.ptr, vs, T, Hkv, D, cap, p0, kc.ptr, vc.ptr), "kv_store")

    def q35_kv_store(self, k, ks, v, vs, T, Hkv, D, cap, p0, kc, vc):
        if T > 0:
            _need(k, ((T - 1) * ks + Hkv * D) * 4, "kv_store k")
            _need(v, ((T - 1) * vs + Hkv * D) * 4, "kv_store v")
        _need(kc, self.cache_bytes(0, Hkv, cap, D), "kv_store key cache")
        _need(vc, self.cache_bytes(0, Hkv, cap, D), "kv_store value cache")
        self.ok(self.k.q35_kv_store(self.raw(), k.ptr, ks, v.ptr, vs, T, Hkv, D, cap, p0, kc.ptr, vc.ptr), "kv_store")

    def q35_kv_store_q(self, kt, k, ks, v, vs, T, Hkv, D, cap, p0, kc, vc):
        if T > 0:
            _need(k, ((T - 1) * ks + Hkv * D) * 4, "kv_store_q k")
            _need(v, ((T - 1) * vs + Hkv * D) * 4, "kv_store_q v")
        if kt in (1, 2):
            _need(kc, self.cache_bytes(kt, Hkv, cap, D), "kv_store_q key cache")
            _need(vc, self.cache_bytes(kt, Hkv, cap, D), "kv_store_q value cache")
        self.ok(self.k.q35_kv_store_q(self.raw(), kt, k.ptr, ks, v.ptr, vs, T, Hkv, D, cap, p0, kc.ptr, vc.ptr), "kv_store_q")

    def mg_kv_store(self, k, v, T, Hkv, D, cap, p0, kc, vc):
        _need(k, T * Hkv * D * 4, "kv_store k")
        _need(v, T * Hkv * D * 4, "kv_store v")
        _need(kc, self.cache_bytes(0, Hkv, cap, D), "kv_store key cache")
        _need(vc, self.cache_bytes(0, Hkv, cap, D), "kv_store value cache")
        self.ok(self.k.mg_kv_store(self.raw(), k.ptr, v.ptr, T, Hkv, D, cap, p0, kc.ptr, vc.ptr), "kv_store")

    def rc_kv_store(self, k, ks, v, vs, T, Hkv, D, R, p0, kc, vc):
        """ns_rc_kv_store: half rows into a ring of R rows a head (position p in slot p % R)."""
        if T > 0:
            _need(k, ((T - 1) * ks + Hkv * D) * 4, "kv_store k")
            _need(v, ((T - 1) * vs + Hkv * D) * 4, "kv_store v")
        _need(kc, self.cache_bytes(0, Hkv, R, D), "kv_store key cache")
        _need(vc, self.cache_bytes(0, Hkv, R, D), "kv_store value cache")
        self.ok(self.k.rc_kv_store(self.raw(), k.ptr, ks, v.ptr, vs, T, Hkv, D, R, p0, kc.ptr, vc.ptr), "kv_store")

    def nh_kv_store(self, k, ks, v, vs, T, Hkv, D, cap, p0, kc, vc):
        if T > 0:
            _need(k, ((T - 1) * ks + Hkv * D) * 4, "kv_store k")
            _need(v, ((T - 1) * vs + Hkv * D) * 4, "kv_store v")
        _need(kc, self.cache_bytes(0, Hkv, cap, D), "kv_store key cache")
        _need(vc, self.cache_bytes(0, Hkv, cap, D), "kv_store value cache")
        self.ok(self.k.nh_kv_store(self.raw(), k.ptr, ks, v.ptr, vs, T, Hkv, D, cap, p0, kc.ptr, vc.ptr), "kv_store")

    def kv_dequant(self, kt, rows, n, D, out):
        rb = kv_row_bytes(kt, D)
        _need(rows, n * rb, "kv_dequant rows")
        _need(out, n * D * 4, "kv_dequant out")
        self.ok(self.k.attn_kv_dequant(self.raw(), kt, rows.ptr, n, D, rb, out.ptr), "kv_dequant")

    def kv_rows_copy(self, src, scap, sbase, dst, dcap, dbase, heads, row_bytes, pos_from, pos_to):
        """Positions [pos_from, pos_to) of every head from one cache geometry into another (slot = (p - base) % cap)."""
        _need(src, heads * scap * row_bytes, "kv_rows_copy source")
        _need(dst, heads * dcap * row_bytes, "kv_rows_copy destination")
        self.ok(self.k.attn_kv_rows_copy(self.raw(), src.ptr, scap, sbase, dst.ptr, dcap, dbase, heads, row_bytes, pos_from, pos_to), "kv_rows_copy")

    def fwht32(self, x, rows, n, stride):
        if rows > 0:
            _need(x, ((rows - 1) * stride + n) * 4, "fwht32 x")
        self.ok(self.k.q35_fwht32(self.raw(), x.ptr, rows, n, stride), "fwht32")

    # ---- decode / verify
    def decode_scratch(self, T, Hq, Hkv, D, p0, win=0):
        return self.k.attn_decode_scratch(T, Hq, Hkv, D, p0, win)

    def decode(self, qt, kt, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, out, scratch, win=0, pm=False, scale=0.0):
        """Typed split-K decode of T rows (ns_attn_decode_t)."""
        if T > 0:
            _need(q, ((T - 1) * qs + Hq * D) * ELT[qt], "decode q")
            _need(out, T * Hq * D * ELT[qt], "decode out")
            _need(scratch, self.decode_scratch(T, Hq, Hkv, D, p0, win) * 4, "decode scratch")
        _need(kc, self.cache_bytes(kt, Hkv, cap, D), "decode key cache")
        _need(vc, self.cache_bytes(kt, Hkv, cap, D), "decode value cache")
        self.ok(self.k.attn_decode_t(self.raw(), qt, kt, int(pm), q.ptr, qs, kc.ptr, vc.ptr, T, Hq, Hkv, D, cap, p0, win, scale, out.ptr,
                                     scratch.ptr if scratch is not None else None), "attention decode")

    def decode_static(self, qt, kt, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, out, win=0, pm=False, scale=0.0):
        """ns_attn_decode_static: the typed decode with the partials in the library's device-resident array - no scratch
        buffer, no allocation."""
        if T > 0:
            _need(q, ((T - 1) * qs + Hq * D) * ELT[qt], "decode q")
            _need(out, T * Hq * D * ELT[qt], "decode out")
        _need(kc, self.cache_bytes(kt, Hkv, cap, D), "decode key cache")
        _need(vc, self.cache_bytes(kt, Hkv, cap, D), "decode value cache")
        self.ok(self.k.attn_decode_static(self.raw(), qt, kt, int(pm), q.ptr, qs, kc.ptr, vc.ptr, T, Hq, Hkv, D, cap, p0, win, scale, out.ptr),
                "attention decode (static scratch)")

    def q35_attn_decode_kv(self, kt, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, out, scratch):
        if T > 0:
            _need(q, ((T - 1) * qs + Hq * D) * 4, "decode q")
            _need(out, T * Hq * D * 4, "decode out")
        if kt in (0, 1, 2):
            _need(kc, self.cache_bytes(kt, Hkv, cap, D), "decode key cache")
            _need(vc, self.cache_bytes(kt, Hkv, cap, D), "decode value cache")
        sc = self.k.q35_attn_decode_scratch(T, Hq, Hkv, D, p0)
        if scratch is not None:
            _need(scratch, sc * 4, "decode scratch")
        self.ok(self.k.q35_attn_decode_kv(self.raw(), kt, q.ptr, qs, kc.ptr, vc.ptr, T, Hq, Hkv, D, cap, p0, out.ptr,
                                          scratch.ptr if scratch is not None else None), "attention decode")

    def mg_attn_decode(self, q, kc, vc, T, Hq, Hkv, D, cap, p0, win, out, scratch):
        _need(q, T * Hq * D * 4, "decode q")
        _need(out, T * Hq * D * 4, "decode out")
        _need(kc, self.cache_bytes(0, Hkv, cap, D), "decode key cache")
        _need(vc, self.cache_bytes(0, Hkv, cap, D), "decode value cache")
        if scratch is not None:
            _need(scratch, self.k.mg_attn_decode_scratch(T, Hq, Hkv, D, p0, win) * 4, "decode scratch")
        self.ok(self.k.mg_attn_decode(self.raw(), q.ptr, kc.ptr, vc.ptr, T, Hq, Hkv, D, cap, p0, win, out.ptr,
                                      scratch.ptr if scratch is not None else None), "attention decode")

    # ---- prompt
    def prompt(self, qt, kt, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, out, win=0, pm=False, scale=0.0):
        """Typed causal flash attention of T prompt rows (ns_attn_prompt_t)."""
        if T > 0:
            _need(q, ((T - 1) * qs + Hq * D) * ELT[qt], "prompt q")
            _need(out, T * Hq * D * ELT[qt], "prompt out")
        _need(kc, self.cache_bytes(kt, Hkv, cap, D), "prompt key cache")
        _need(vc, self.cache_bytes(kt, Hkv, cap, D), "prompt value cache")
        self.ok(self.k.attn_prompt_t(self.raw(), qt, kt, int(pm), q.ptr, qs, kc.ptr, vc.ptr, T, Hq, Hkv, D, cap, p0, win, scale, out.ptr),
                "attention prompt")

    def mg_attn_prompt(self, q, kc, vc, T, Hq, Hkv, D, cap, p0, win, out):
        _need(q, T * Hq * D * 4, "prompt q")
        _need(out, T * Hq * D * 4, "prompt out")
        _need(kc, self.cache_bytes(0, Hkv, cap, D), "prompt key cache")
        _need(vc, self.cache_bytes(0, Hkv, cap, D), "prompt value cache")
        self.ok(self.k.mg_attn_prompt(self.raw(), q.ptr, kc.ptr, vc.ptr, T, Hq, Hkv, D, cap, p0, win, out.ptr), "attention prompt")

    # ---- the engines' own entry points
    def mg_attn(self, q, kc, vc, T, Hq, Hkv, D, cap, p0, win, causal, out, scratch):
        _need(q, T * Hq * D * 4, "attention q")
        _need(out, T * Hq * D * 4, "attention out")
        _need(kc, self.cache_bytes(0, Hkv, cap, D), "attention key cache")
        _need(vc, self.cache_bytes(0, Hkv, cap, D), "attention value cache")
        if scratch is not None:
            _need(scratch, self.k.mg_attn_scratch(T, Hq, Hkv, D, p0, win, int(causal)) * 4, "attention scratch")
        self.ok(self.k.mg_attn(self.raw(), q.ptr, kc.ptr, vc.ptr, T, Hq, Hkv, D, cap, p0, win, int(causal), out.ptr,
                               scratch.ptr if scratch is not None else None), "attention")

    def rc_attn(self, q, qs, kc, vc, T, Hq, Hkv, D, R, W, p0, out, scratch):
        """ns_rc_attn: ricursive's attention over a ring of R rows a head, window W (0: none)."""
        if T > 0:
            _need(q, ((T - 1) * qs + Hq * D) * 4, "attention q")
            _need(out, T * Hq * D * 4, "attention out")
        _need(kc, self.cache_bytes(0, Hkv, R, D), "attention key cache")
        _need(vc, self.cache_bytes(0, Hkv, R, D), "attention value cache")
        if scratch is not None:
            _need(scratch, self.k.rc_attn_scratch(T, Hq, Hkv, D, W, p0) * 4, "attention scratch")
        self.ok(self.k.rc_attn(self.raw(), q.ptr, qs, kc.ptr, vc.ptr, T, Hq, Hkv, D, R, W, p0, out.ptr,
                               scratch.ptr if scratch is not None else None), "attention")

    def rc_flash(self, q, kc, vc, T, Hq, Hkv, D, cap, p0, win, out, scratch=None):
        """ricursive's silo names: ns_rc_flash_decode (1..16 rows, with scratch) or ns_rc_flash_prompt (more)."""
        _need(q, T * Hq * D * 4, "attention q")
        _need(out, T * Hq * D * 4, "attention out")
        _need(kc, self.cache_bytes(0, Hkv, cap, D), "attention key cache")
        _need(vc, self.cache_bytes(0, Hkv, cap, D), "attention value cache")
        if T <= 16:
            if scratch is not None:
                _need(scratch, max(0, self.k.rc_flash_decode_scratch(T, Hq, Hkv, D, p0, win)) * 4, "attention scratch")
            self.ok(self.k.rc_flash_decode(self.raw(), q.ptr, kc.ptr, vc.ptr, T, Hq, Hkv, D, cap, p0, win, out.ptr,
                                           scratch.ptr if scratch is not None else None), "attention")
        else:
            self.ok(self.k.rc_flash_prompt(self.raw(), q.ptr, kc.ptr, vc.ptr, T, Hq, Hkv, D, cap, p0, win, out.ptr), "attention")

    def nh_attn(self, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, out, scratch):
        """ns_nh_attn: nemotron-h's attention layers (causal, no window)."""
        if T > 0:
            _need(q, ((T - 1) * qs + Hq * D) * 4, "attention q")
            _need(out, T * Hq * D * 4, "attention out")
        _need(kc, self.cache_bytes(0, Hkv, cap, D), "attention key cache")
        _need(vc, self.cache_bytes(0, Hkv, cap, D), "attention value cache")
        if scratch is not None:
            _need(scratch, self.k.nh_attn_scratch(T, Hq, Hkv, D, p0) * 4, "attention scratch")
        self.ok(self.k.nh_attn(self.raw(), q.ptr, qs, kc.ptr, vc.ptr, T, Hq, Hkv, D, cap, p0, out.ptr,
                               scratch.ptr if scratch is not None else None), "attention")

    def mg_attn_block(self, q, kc, vc, T, Hq, Hkv, D, cap, p0, win, out, scratch):
        """ns_mg_attn_block: the drafter's block (not causal)."""
        _need(q, T * Hq * D * 4, "block q")
        _need(out, T * Hq * D * 4, "block out")
        _need(kc, self.cache_bytes(0, Hkv, cap, D), "block key cache")
        _need(vc, self.cache_bytes(0, Hkv, cap, D), "block value cache")
        if scratch is not None:
            _need(scratch, self.k.mg_attn_block_scratch(T, Hq, Hkv, D, p0, win) * 4, "block scratch")
        self.ok(self.k.mg_attn_block(self.raw(), q.ptr, kc.ptr, vc.ptr, T, Hq, Hkv, D, cap, p0, win, out.ptr,
                                     scratch.ptr if scratch is not None else None), "attention block")

    def q35_attn_probs(self, kt, q, kc, Hq, Hkv, D, cap, n, mode, scratch, out):
        """ns_q35_attn_probs: out [n] += the heads' weights of every key (mode 0 their mean, 1 their largest)."""
        _need(q, Hq * D * 4, "attn_probs q")
        _need(kc, self.cache_bytes(kt, Hkv, cap, D), "attn_probs key cache")
        _need(scratch, 2 * Hq * 4, "attn_probs scratch")
        _need(out, n * 4, "attn_probs out")
        self.ok(self.k.q35_attn_probs(self.raw(), kt, q.ptr, kc.ptr, Hq, Hkv, D, cap, n, mode, scratch.ptr, out.ptr), "attn_probs")

    def q35_attn(self, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, out, scratch):
        if T > 0:
            _need(q, ((T - 1) * qs + Hq * D) * 4, "attention q")
            _need(out, T * Hq * D * 4, "attention out")
        _need(kc, self.cache_bytes(0, Hkv, cap, D), "attention key cache")
        _need(vc, self.cache_bytes(0, Hkv, cap, D), "attention value cache")
        if scratch is not None:
            _need(scratch, self.k.q35_attn_scratch(T, Hq, Hkv, D, p0) * 4, "attention scratch")
        self.ok(self.k.q35_attn(self.raw(), q.ptr, qs, kc.ptr, vc.ptr, T, Hq, Hkv, D, cap, p0, out.ptr,
                                scratch.ptr if scratch is not None else None), "attention")

    # ---- MLA (include/ns_mla.h; wrappers as llm/deepseek2/src/ops.rs:409-445)
    def mla_latent_scratch(self, T, H, pos0):
        return self.k.mla_decode_latent_scratch(T, H, pos0)

    def mla_decode_latent(self, qt, qa, cache, u, T, H, R, pos0, scale, scratch):
        """qa [T][H][512 + R] (absorbed) over the cache's cells 0 .. pos0 + T - 1 -> u [T][H][512]."""
        e = ELT[qt]
        _need(qa, T * H * (512 + R) * e, "mla_decode_latent qa")
        _need(cache, (pos0 + T) * (512 + R) * 2, "mla_decode_latent cache")
        _need(u, T * H * 512 * e, "mla_decode_latent u")
        _need(scratch, self.mla_latent_scratch(T, H, pos0) * 4, "mla_decode_latent scratch")
        self.ok(self.k.mla_decode_latent(self.raw(), qt, qa.ptr, cache.ptr, u.ptr, T, H, R, pos0, scale, scratch.ptr), "mla_decode_latent")

    def mla_decode(self, q, kb, vb, cache, out, T, H, pos0, scale):
        """ns_ds2_mla_decode: q [T][H][192], k_b / v_b half, cache half [.., 576] -> out [T][H][128]."""
        _need(q, T * H * 192 * 4, "mla_decode q")
        _need(kb, H * 512 * 128 * 2, "mla_decode k_b")
        _need(vb, H * 128 * 512 * 2, "mla_decode v_b")
        _need(cache, (pos0 + T) * 576 * 2, "mla_decode cache")
        _need(out, T * H * 128 * 4, "mla_decode out")
        self.ok(self.k.ds2_mla_decode(self.raw(), q.ptr, kb.ptr, vb.ptr, cache.ptr, out.ptr, T, H, pos0, scale), "mla_decode")

    def mla_decode_q6k(self, q, kvb, cache, out, T, H, pos0, scale):
        """ns_ds2_mla_decode_q6k: q [T][H][192], kv_b as Q6_K rows ([H][256] rows of 420 bytes), cache half [.., 576] -> out [T][H][128]."""
        _need(q, T * H * 192 * 4, "mla_decode_q6k q")
        _need(kvb, H * 256 * 420, "mla_decode_q6k kv_b")
        _need(cache, (pos0 + T) * 576 * 2, "mla_decode_q6k cache")
        _need(out, T * H * 128 * 4, "mla_decode_q6k out")
        self.ok(self.k.ds2_mla_decode_q6k(self.raw(), q.ptr, kvb.ptr, cache.ptr, out.ptr, T, H, pos0, scale), "mla_decode_q6k")

    def ds2_kv_store(self, kv, w, eps, cache, T, L, R, pos0, freq_base, freq_scale, ext_factor, mscale, corr0, corr1):
        _need(kv, T * (L + R) * 4, "kv_store kv")
        _need(w, L * 4, "kv_store w")
        _need(cache, (pos0 + T) * (L + R) * 2, "kv_store cache")
        self.ok(self.k.ds2_kv_store(self.raw(), kv.ptr, w.ptr, eps, cache.ptr, T, L, R, pos0, freq_base, freq_scale, ext_factor, mscale, corr0, corr1),
                "kv_store")

    def mla_attend(self, qa, c, u, T, H, L, pos0, scale, q8=False, sel=None, sel_cnt=None, K=0):
        """GLM's latent-only MLA: ns_mla_attend_sel / ns_mla_attend_sel_q8; sel [T][K] pools and sel_cnt [T], or dense."""
        _need(qa, T * H * L * 4, "mla_attend qa")
        _need(c, (pos0 + T) * ((L // 32 * 2 + L) if q8 else 2 * L), "mla_attend cache")
        _need(u, T * H * L * 4, "mla_attend u")
        if sel_cnt is not None:
            _need(sel, T * K * 4, "mla_attend pools")
            _need(sel_cnt, T * 4, "mla_attend pool counts")
        f = self.k.mla_attend_sel_q8 if q8 else self.k.mla_attend_sel
        opt = lambda b: b.ptr if b is not None else None
        self.ok(f(self.raw(), qa.ptr, c.ptr, u.ptr, T, H, L, pos0, scale, opt(sel), opt(sel_cnt), K), "mla_attend")

    def mla_attend_f32(self, qa, c, u, T, H, L, pos0, scale):
        """ns_mla_attend: the dense form over a float32 latent cache [n][L]."""
        _need(qa, T * H * L * 4, "mla_attend qa")
        _need(c, (pos0 + T) * L * 4, "mla_attend cache")
        _need(u, T * H * L * 4, "mla_attend u")
        self.ok(self.k.mla_attend(self.raw(), qa.ptr, c.ptr, u.ptr, T, H, L, pos0, scale), "mla_attend")

    def gather_q8_h(self, src, rows, idx, out, n, L):
        """ns_gather_q8_h: out [n][L] half = the q8 latent rows idx[i] of src (`rows` of them), widened."""
        _need(src, rows * (L // 32 * 2 + L), "gather_q8_h rows")
        _need(idx, n * 4, "gather_q8_h indices")
        _need(out, n * L * 2, "gather_q8_h out")
        self.ok(self.k.gather_q8_h(self.raw(), src.ptr, idx.ptr, out.ptr, n, L), "gather_q8_h")

    def mla_cells(self, T, K, pos0, idx, n, NC, sel=None, sel_cnt=None):
        """ns_mla_cells: each row's cells as a list idx [T][NC] int32 and their count n [T] (sel / sel_cnt None: every
        cell up to the row's position)."""
        _need(idx, T * NC * 4, "mla_cells idx")
        _need(n, T * 4, "mla_cells counts")
        if sel_cnt is not None:
            _need(sel, T * K * 4, "mla_cells pools")
            _need(sel_cnt, T * 4, "mla_cells pool counts")
        opt = lambda b: b.ptr if b is not None else None
        self.ok(self.k.mla_cells(self.raw(), opt(sel), opt(sel_cnt), T, K, pos0, idx.ptr, n.ptr, NC), "mla_cells")

    def softmax_masked(self, S, R, H, NC, n, scale):
        """ns_softmax_masked: S [R H][NC] float32 in place, row r's heads over their first n[r] cells, 0 behind."""
        _need(S, R * H * NC * 4, "softmax_masked scores")
        _need(n, R * 4, "softmax_masked counts")
        self.ok(self.k.softmax_masked(self.raw(), S.ptr, R, H, NC, n.ptr, scale), "softmax_masked")

    def gather_h(self, src, rows, idx, out, n, C):
        """ns_gather_h: out [n][C] half = the rows idx[i] of src (`rows` of them)."""
        _need(src, rows * C * 2, "gather_h rows")
        _need(idx, n * 4, "gather_h indices")
        _need(out, n * C * 2, "gather_h out")
        self.ok(self.k.gather_h(self.raw(), src.ptr, idx.ptr, out.ptr, n, C), "gather_h")

    def to_f16(self, x, y, n):
        """ns_to_f16: y [n] half = x [n] float32."""
        _need(x, n * 4, "to_f16 x")
        _need(y, n * 2, "to_f16 y")
        self.ok(self.k.to_f16(self.raw(), x.ptr, y.ptr, n), "to_f16")

    def gemm_f16(self, T, N, K, x, ldx, w, y, ldy, accumulate=False):
        """ns_gemm_f16: y [T, N] float32 (+)= x [T, K] half . w [N, K]^T half (kernels/llm/glm5next/glm.cpp:217-225)."""
        self.gemm_batch_h(1, True, T, N, K, x, ldx, 0, w, K, 0, y, ldy, 0, accumulate, _one=True)

    def gemm_batch_h(self, batch, trans_w, T, N, K, x, ldx, sx, w, ldw, sw, y, ldy, sy, accumulate=False, _one=False):
        """ns_gemm_batch_h: `batch` products y_b [T, N] float32 (+)= x_b [T, K] . op(w_b), half operands; op(w) = w^T (w
        [N, K]) with trans_w, else w ([K, N]); strides in elements (kernels/llm/glm5next/glm.cpp:265-276)."""
        if batch > 0 and T > 0 and N > 0:
            _need(x, ((batch - 1) * sx + (T - 1) * ldx + K) * 2, "gemm x")
            _need(w, ((batch - 1) * sw + ((N if trans_w else K) - 1) * ldw + (K if trans_w else N)) * 2, "gemm w")
            _need(y, ((batch - 1) * sy + (T - 1) * ldy + N) * 4, "gemm y")
        if _one:
            self.ok(self.k.gemm_f16(self.raw(), T, N, K, x.ptr, ldx, w.ptr, y.ptr, ldy, int(accumulate)), "gemm_f16")
        else:
            self.ok(self.k.gemm_batch_h(self.raw(), batch, int(trans_w), T, N, K, x.ptr, ldx, sx, w.ptr, ldw, sw, y.ptr, ldy, sy,
                                        int(accumulate)), "gemm_batch_h")

    def to_q8row(self, x, y, n, L):
        _need(x, n * L * 4, "to_q8row x")
        _need(y, n * (L // 32 * 2 + L), "to_q8row y")
        self.ok(self.k.to_q8row(self.raw(), x.ptr, y.ptr, n, L), "to_q8row")

    def minimaxm3_attend(self, q, kc, vc, out, T, H, G, pos0, scale, sel=None, K=0):
        _need(q, T * H * 128 * 4, "attend q")
        _need(out, T * H * 128 * 4, "attend out")
        _need(kc, (pos0 + T) * G * 128 * 2, "attend key cache")
        _need(vc, (pos0 + T) * G * 128 * 2, "attend value cache")
        if sel is not None:
            _need(sel, T * G * K * 4, "attend block lists")
        self.ok(self.k.llm_minimaxm3_attend(self.raw(), q.ptr, kc.ptr, vc.ptr, sel.ptr if sel is not None else None, K, out.ptr, T, H, G, pos0, scale),
                "attend")

    def mm3s_attend(self, form, q, kc, vc, out, T, H, G, pos0, scale, sel=None, K=0, S=0, part=None, w0=0):
        """The MiniMax silo's names: form "", "x", "split", "x_split" or "block" (ns_mm3s_attend*)."""
        _need(q, T * H * 128 * 4, "attend q")
        _need(out, T * H * 128 * 4, "attend out")
        _need(kc, (pos0 + T) * G * 128 * 2, "attend key cache")
        _need(vc, (pos0 + T) * G * 128 * 2, "attend value cache")
        if sel is not None:
            _need(sel, T * G * K * 4, "attend block lists")
        if form in ("split", "x_split", "block"):
            _need(part, T * G * S * 16 * 130 * 4, "attend partials")
        sp = sel.ptr if sel is not None else None
        if form == "block":
            rc = self.k.mm3s_attend_block(self.raw(), q.ptr, kc.ptr, vc.ptr, out.ptr, T, H, G, pos0, w0, S, part.ptr)
        elif form in ("split", "x_split"):
            rc = getattr(self.k, "mm3s_attend_" + form)(self.raw(), q.ptr, kc.ptr, vc.ptr, sp, K, out.ptr, T, H, G, pos0, scale, S, part.ptr)
        else:
            rc = getattr(self.k, "mm3s_attend" + ("_x" if form == "x" else ""))(self.raw(), q.ptr, kc.ptr, vc.ptr, sp, K, out.ptr, T, H, G, pos0, scale)
        self.ok(rc, "mm3s_attend" + ("_" + form if form else ""))

    def minimaxm3_idx_scores(self, iq, ik, bs, T, G, nblk, pos0, local):
        _need(iq, T * G * 128 * 4, "idx_scores iq")
        _need(ik, (pos0 + T) * 128 * 2, "idx_scores ik")
        _need(bs, T * G * nblk * 4, "idx_scores scores")
        self.ok(self.k.llm_minimaxm3_idx_scores(self.raw(), iq.ptr, ik.ptr, bs.ptr, T, G, nblk, pos0, local), "idx_scores")

    def minimaxm3_idx_topk(self, bs, sel, T, G, nblk, K):
        _need(bs, T * G * nblk * 4, "idx_topk scores")
        _need(sel, T * G * K * 4, "idx_topk lists")
        self.ok(self.k.llm_minimaxm3_idx_topk(self.raw(), bs.ptr, sel.ptr, T, G, nblk, K), "idx_topk")

    # ---- the step in front of attention: norm, rotary positions, store
    def q35_qk_norm_rope(self, src, ss, hs, dst, ds, T, H, D, w, eps, n_rot, theta, p0, pos3=None, sections=(0, 0, 0)):
        """ns_q35_qk_norm_rope (pos3 None) / ns_q35_qk_norm_rope_pos / ns_q35_rope (w None): float32 rows."""
        _need(src, ((T - 1) * ss + (H - 1) * hs + D) * 4, "qk_norm_rope src")
        _need(dst, ((T - 1) * ds + H * D) * 4, "qk_norm_rope dst")
        if w is None:
            return self.ok(self.k.q35_rope(self.raw(), src.ptr, ss, hs, dst.ptr, ds, T, H, D, n_rot, theta, p0), "q35_rope")
        _need(w, D * 4, "qk_norm_rope weight")
        if pos3 is None:
            return self.ok(self.k.q35_qk_norm_rope(self.raw(), src.ptr, ss, hs, dst.ptr, ds, T, H, D, w.ptr, eps, n_rot, theta, p0), "q35_qk_norm_rope")
        _need(pos3, T * 3 * 4, "qk_norm_rope positions")
        self.ok(self.k.q35_qk_norm_rope_pos(self.raw(), src.ptr, ss, hs, dst.ptr, ds, T, H, D, w.ptr, eps, n_rot, theta, pos3.ptr, *sections),
                "q35_qk_norm_rope_pos")

    def mg_qk_norm_rope(self, x, xs, y, ys, T, H, D, w, eps, rope, theta, p0):
        _need(x, ((T - 1) * xs + H * D) * 4, "mg_qk_norm_rope x")
        _need(y, ((T - 1) * ys + H * D) * 4, "mg_qk_norm_rope y")
        _need(w, D * 4, "mg_qk_norm_rope weight")
        self.ok(self.k.mg_qk_norm_rope(self.raw(), x.ptr, xs, y.ptr, ys, T, H, D, w.ptr, eps, rope, theta, p0), "mg_qk_norm_rope")

    def minimaxm3_rope(self, x, T, H, row, head, n_rot, pos0, base):
        _need(x, ((T - 1) * row + H * head) * 4, "minimaxm3_rope x")
        self.ok(self.k.llm_minimaxm3_rope(self.raw(), x.ptr, T, H, row, head, n_rot, pos0, base), "minimaxm3_rope")

    def mm3s_attn_post(self, q, k, v, iq, ik, qn, kn, iqn, ikn, kc, vc, ic, H, G, IH, HD, n_rot, pos, base, eps):
        """kc, vc, ic: (buffer, byte offset of the token's row). iq / ik / iqn / ikn / ic None when IH == 0."""
        _need(q, H * HD * 4, "attn_post q")
        _need(k, G * HD * 4, "attn_post k")
        _need(v, G * HD * 4, "attn_post v")
        _need(qn, HD * 4, "attn_post q weight")
        _need(kn, HD * 4, "attn_post k weight")
        for (b, off), n, what in ((kc, G * HD * 2, "kc"), (vc, G * HD * 2, "vc")) + (((ic, HD * 2, "ic"),) if IH > 0 else ()):
            _need(b, off + n, "attn_post " + what)
        if IH > 0:
            _need(iq, IH * HD * 4, "attn_post iq")
            _need(ik, HD * 4, "attn_post ik")
        opt = lambda b: b.ptr if b is not None else None
        self.ok(self.k.mm3s_attn_post(self.raw(), q.ptr, k.ptr, v.ptr, opt(iq), opt(ik), qn.ptr, kn.ptr, opt(iqn), opt(ikn), kc[0].ptr + kc[1],
                                      vc[0].ptr + vc[1], (ic[0].ptr + ic[1]) if IH > 0 else None, H, G, IH, HD, n_rot, pos, base, eps), "mm3s_attn_post")

    def pre_store(self, rope, qt, kt, ring, q, qss, qhs, qo, qos, k, kss, khs, v, vss, qw, kw, eps, n_rot, theta, T, Hq, Hkv, D, cap, p0, kc, vc):
        """ns_attn_pre_store: q normed + rotated into qo, k normed + rotated + v written into the caches, one launch."""
        _need(q, ((T - 1) * qss + (Hq - 1) * qhs + D) * 4, "pre_store q")
        _need(qo, ((T - 1) * qos + Hq * D) * ELT[qt], "pre_store q out")
        _need(k, ((T - 1) * kss + (Hkv - 1) * khs + D) * 4, "pre_store k")
        _need(v, ((T - 1) * vss + Hkv * D) * 4, "pre_store v")
        _need(qw, D * 4, "pre_store q weight")
        _need(kw, D * 4, "pre_store k weight")
        _need(kc, self.cache_bytes(kt, Hkv, cap, D), "pre_store kc")
        _need(vc, self.cache_bytes(kt, Hkv, cap, D), "pre_store vc")
        self.ok(self.k.attn_pre_store(self.raw(), rope, qt, kt, int(ring), q.ptr, qss, qhs, qo.ptr, qos, k.ptr, kss, khs, v.ptr, vss, qw.ptr, kw.ptr, eps,
                                      n_rot, theta, T, Hq, Hkv, D, cap, p0, kc.ptr, vc.ptr), "pre_store")
