// attn_api.cpp: the reference engines' attention entry points (ns_q35_*, ns_mg_*, ns_llm_minimaxm3_attend) routed to the
// two kernels of this library: the split-K decode kernel for passes of 1..16 rows, the flash prefill kernel for longer
// ones. Names, arguments and error behaviour follow the reference headers cited in ns_attn.h; zero-row calls return 0
// before anything is checked, as the reference's do (kernels/llm/qwen35/q35.cpp:598).
#include "ns_internal.hpp"
#include "ns_attn.h"
#include "ns_pre.h"

#include "attn_host.hpp"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdlib>

namespace {
}

extern "C" {

// ---- prompt form ------------------------------------------------------------------------------------------------------

int ns_mg_attn_prompt_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D) {
    return T > DECODE_ROWS && (D == 128 || D == 256) && Hkv > 0 && Hq > 0 && Hq % Hkv == 0;
}

int ns_mg_attn_prompt(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap,
                      int64_t p0, int64_t win, float* out) {
    if (!ns_mg_attn_prompt_supported(T, Hq, Hkv, D)) return ns_fail("ns_mg_attn_prompt: more than 16 rows, heads of 128 or 256, query heads a multiple of the key heads");
    return ns_attn_prompt_any(g, "ns_mg_attn_prompt", 0, 0, 0, q, Hq * D, kc, vc, T, Hq, Hkv, D, cap, p0, win, 1, -1, 0.0f, out);
}

int ns_q35_attn_prompt_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D) { return ns_mg_attn_prompt_supported(T, Hq, Hkv, D); }

int ns_q35_attn_prompt(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D,
                       int64_t cap, int64_t p0, float* out) {
    if (!ns_q35_attn_prompt_supported(T, Hq, Hkv, D)) return ns_fail("ns_q35_attn_prompt: more than 16 rows, heads of 128 or 256, query heads a multiple of the key heads");
    return ns_attn_prompt_any(g, "ns_q35_attn_prompt", 0, 0, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, 1, -1, 0.0f, out);
}

int ns_q35_attn_prompt_kv(ns_gpu* g, int kt, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv,
                          int64_t D, int64_t cap, int64_t p0, float* out) {
    if (!ns_q35_attn_prompt_supported(T, Hq, Hkv, D)) return ns_fail("ns_q35_attn_prompt_kv: more than 16 rows, heads of 128 or 256, query heads a multiple of the key heads");
    if (kt < 0 || kt > 2) return ns_fail("ns_q35_attn_prompt_kv: a cache form 0 (half), 1 (q8_0) or 2 (q4_0)");
    return ns_attn_prompt_any(g, "ns_q35_attn_prompt_kv", 0, kt, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, 1, -1, 0.0f, out);
}

int ns_nhs_attn_prompt_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D) { return ns_mg_attn_prompt_supported(T, Hq, Hkv, D); }

int ns_nhs_attn_prompt(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D,
                       int64_t cap, int64_t p0, float* out) {
    if (!ns_nhs_attn_prompt_supported(T, Hq, Hkv, D)) return ns_fail("ns_nhs_attn_prompt: more than 16 rows, heads of 128 or 256, query heads a multiple of the key heads");
    return ns_attn_prompt_any(g, "ns_nhs_attn_prompt", 0, 0, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, 1, -1, 0.0f, out);
}

// ---- the engines' own entry points: decode rows split, prompt rows flash -------------------------------------------------

int64_t ns_q35_attn_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0) {
    return T >= 1 && T <= DECODE_ROWS ? ns_attn_decode_scratch(T, Hq, Hkv, D, p0, 0) : 0;
}

int ns_q35_attn(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D,
                int64_t cap, int64_t p0, float* out, float* scratch) {
    if (T <= 0) return 0;
    if (p0 + T > cap) return ns_fail("ns_q35_attn: past the cache's capacity");
    if (T <= DECODE_ROWS) return ns_attn_decode_any(g, "ns_q35_attn", 0, 0, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, DecodeExtra{}, 0.0f, out, scratch);
    return ns_attn_prompt_any(g, "ns_q35_attn", 0, 0, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, 1, -1, 0.0f, out);
}

int64_t ns_mg_attn_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0, int64_t win, int causal) {
    (void) causal;
    return T >= 1 && T <= DECODE_ROWS ? ns_attn_decode_scratch(T, Hq, Hkv, D, p0, win) : 0;
}

int ns_mg_attn(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0,
               int64_t win, int causal, float* out, float* scratch) {
    if (T <= 0) return 0;
    DecodeExtra x;
    x.causal = causal ? 1 : 0;
    if (T <= DECODE_ROWS) return ns_attn_decode_any(g, "ns_mg_attn", 0, 0, 0, q, Hq * D, kc, vc, T, Hq, Hkv, D, cap, p0, win, x, 0.0f, out, scratch);
    return ns_attn_prompt_any(g, "ns_mg_attn", 0, 0, 0, q, Hq * D, kc, vc, T, Hq, Hkv, D, cap, p0, win, x.causal, -1, 0.0f, out);
}

// the drafter's block: rows p0 .. p0 + T - 1 each seeing its window's first key .. the block's last (not causal)
int64_t ns_mg_attn_block_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0, int64_t win) {
    return T >= 1 && T <= DECODE_ROWS ? ns_attn_decode_scratch(T, Hq, Hkv, D, p0, win) : 0;
}

int ns_mg_attn_block(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0,
                     int64_t win, float* out, float* scratch) {
    if (T < 1) return ns_fail("ns_mg_attn_block: at least one row");
    return ns_mg_attn(g, q, kc, vc, T, Hq, Hkv, D, cap, p0, win, 0, out, scratch);
}

// ---- ricursive and nemotron-h: the same two kernels under their engines' names -----------------------------------------

int64_t ns_rc_attn_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t W, int64_t p0) {
    return T >= 1 && T <= DECODE_ROWS ? ns_attn_decode_scratch(T, Hq, Hkv, D, p0, W) : 0;
}

int ns_rc_attn(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t R,
               int64_t W, int64_t p0, float* out, float* scratch) {
    if (T <= 0) return 0;
    if (W > 0 && R < W + T - 1 && p0 + T > R) return ns_fail("ns_rc_attn: the ring is smaller than the window and the rows");
    if (W == 0 && p0 + T > R) return ns_fail("ns_rc_attn: past the cache's capacity");
    if (D != 128) return ns_fail("ns_rc_attn: heads of 128");
    const int64_t G = Hkv > 0 && Hq % Hkv == 0 ? Hq / Hkv : 0;
    if (G != 1 && G != 2 && G != 4 && G != 6 && G != 8 && G != 10) return ns_fail("ns_rc_attn: 1, 2, 4, 6, 8 or 10 query heads a key head");
    if (T <= DECODE_ROWS) return ns_attn_decode_any(g, "ns_rc_attn", 0, 0, 0, q, qs, kc, vc, T, Hq, Hkv, D, R, p0, W, DecodeExtra{}, 0.0f, out, scratch);
    return ns_attn_prompt_any(g, "ns_rc_attn", 0, 0, 0, q, qs, kc, vc, T, Hq, Hkv, D, R, p0, W, 1, -1, 0.0f, out);
}

// ricursive's silo names (kernels/llm/ricursive/silo/attn.cpp:282-360): heads of 128, 10 query heads a key head, ring
// caches, a window; rows Hq x 128 floats apart
int ns_rc_flash_decode_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D) { return T >= 1 && T <= DECODE_ROWS && D == 128 && Hkv > 0 && Hq == 10 * Hkv; }

int64_t ns_rc_flash_decode_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0, int64_t win) {
    return ns_attn_decode_scratch(T, Hq, Hkv, D, p0, win);
}

int ns_rc_flash_decode(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0,
                       int64_t win, float* out, float* scratch) {
    if (!ns_rc_flash_decode_supported(T, Hq, Hkv, D)) return ns_fail("ns_rc_flash_decode: 1..16 rows, heads of 128, 10 query heads a key head");
    if (!scratch) return ns_fail("ns_rc_flash_decode: no scratch");
    return ns_attn_decode_any(g, "ns_rc_flash_decode", 0, 0, 0, q, Hq * D, kc, vc, T, Hq, Hkv, D, cap, p0, win, DecodeExtra{}, 0.0f, out, scratch);
}

int ns_rc_flash_prompt_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D) { return T > DECODE_ROWS && D == 128 && Hkv > 0 && Hq == 10 * Hkv; }

int ns_rc_flash_prompt(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0,
                       int64_t win, float* out) {
    if (!ns_rc_flash_prompt_supported(T, Hq, Hkv, D)) return ns_fail("ns_rc_flash_prompt: more than 16 rows, heads of 128, 10 query heads a key head");
    const int64_t need = win > 0 ? std::min(p0 + T, win + T - 1) : p0 + T;
    if (need > cap) return ns_fail("ns_rc_flash_prompt: the cache's ring is shorter than the window and the pass");
    return ns_attn_prompt_any(g, "ns_rc_flash_prompt", 0, 0, 0, q, Hq * D, kc, vc, T, Hq, Hkv, D, cap, p0, win, 1, -1, 0.0f, out);
}

int64_t ns_nh_attn_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0) {
    return T >= 1 && T <= DECODE_ROWS ? ns_attn_decode_scratch(T, Hq, Hkv, D, p0, 0) : 0;
}

int ns_nh_attn(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap,
               int64_t p0, float* out, float* scratch) {
    if (T <= 0) return 0;
    if (p0 + T > cap) return ns_fail("ns_nh_attn: past the cache's capacity");
    if (D != 128 || Hkv <= 0 || Hq % 8 != 0 || Hq % Hkv != 0 || (Hq / Hkv) % 8 != 0)
        return ns_fail("ns_nh_attn: head 128, query heads a multiple of 8 a key head");
    if (T <= DECODE_ROWS) return ns_attn_decode_any(g, "ns_nh_attn", 0, 0, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, DecodeExtra{}, 0.0f, out, scratch);
    return ns_attn_prompt_any(g, "ns_nh_attn", 0, 0, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, 1, -1, 0.0f, out);
}

// ---- MiniMax-M3: position-major cache, explicit scale, no scratch argument ------------------------------------------------

// One body for the dense / block-list passes of every MiniMax entry point. part NULL: the partials of a pass of up to 16
// rows go through the library's own scratch; else through the caller's `part` where it holds them (part_floats), the
// library's own otherwise. kfirst >= 0 with causal 0: a draft block (every row sees kfirst .. the block's last key).
static int mm3_attend(ns_gpu* g, const char* who, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K, float* out,
                      int64_t T, int64_t H, int64_t G, int64_t pos0, float scale, int causal, int64_t kfirst, float* part, int64_t part_floats) {
    if (T <= 0) return 0;
    const std::string w(who);
    if (G <= 0 || H <= 0 || H % G) return ns_fail(w + ": heads");
    if (!(scale > 0.0f)) return ns_fail(w + ": a positive scale");
    if (pos0 < 0) return ns_fail(w + ": a position");
    float* sc = g->own_scratch;
    int64_t sc_floats = (int64_t) ns_own_floats(g);
    if (sel) {
        if (part && part_floats >= T * H * K * 130) sc = part, sc_floats = part_floats;      // (splits of at least 128 keys: at most K of them)
        return ns_attn_decode_sel(g, who, q, kc, vc, sel, K, out, T, H, G, pos0, scale, sc, (size_t) sc_floats);
    }
    const int64_t cap = pos0 + T;
    if (T <= DECODE_ROWS) {
        DecodeExtra x;
        x.causal = causal;
        x.kfirst = kfirst;
        // the splits lie at absolute multiples of at least 128 keys: never more than the 128-key blocks the keys touch
        const int64_t worst = T * H * ((cap - 1) / 128 - std::max<int64_t>(kfirst, 0) / 128 + 1) * 130;
        if (part && part_floats >= worst) sc = part, sc_floats = part_floats;
        x.scratch_floats = sc_floats;
        return ns_attn_decode_any(g, who, 0, 0, 1, q, H * 128, kc, vc, T, H, G, 128, cap, pos0, 0, x, scale, out, sc);
    }
    return ns_attn_prompt_any(g, who, 0, 0, 1, q, H * 128, kc, vc, T, H, G, 128, cap, pos0, 0, causal, kfirst, scale, out);
}

int ns_llm_minimaxm3_attend(ns_gpu* g, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K, float* out, int64_t T,
                            int64_t H, int64_t G, int64_t pos0, float scale) {
    return mm3_attend(g, "ns_llm_minimaxm3_attend", q, kc, vc, sel, K, out, T, H, G, pos0, scale, 1, -1, nullptr, 0);
}

// ---- the MiniMax silo's names for the same passes (kernels/llm/minimaxm3/silo/mm3s.h:14-33,61-62). The reference's
// vector-unit and matrix-unit forms are one kernel family here; its split forms take the caller's S = ceil(keys / 128)
// and `part` (T G S 16 130 floats), which always hold this library's partials (splits of at least 128 keys)

int ns_mm3s_attend_supported(int64_t H, int64_t G, int64_t head) { return head == 128 && G > 0 && H > 0 && H % G == 0; }

int ns_mm3s_attend(ns_gpu* g, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K, float* out, int64_t T, int64_t H,
                   int64_t G, int64_t pos0, float scale) {
    return mm3_attend(g, "ns_mm3s_attend", q, kc, vc, sel, K, out, T, H, G, pos0, scale, 1, -1, nullptr, 0);
}

// (the reference's matrix-unit forms ignore `scale` and use 1 / sqrt(128): kernels/llm/minimaxm3/silo/attnx.cpp:40,245;
// here a positive scale is honoured and anything else means 1 / sqrt(128))
static float mm3x_scale(float scale) { return scale > 0.0f ? scale : 0.08838834764831845f; }

int ns_mm3s_attend_x(ns_gpu* g, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K, float* out, int64_t T, int64_t H,
                     int64_t G, int64_t pos0, float scale) {
    return mm3_attend(g, "ns_mm3s_attend_x", q, kc, vc, sel, K, out, T, H, G, pos0, mm3x_scale(scale), 1, -1, nullptr, 0);
}

int ns_mm3s_attend_split(ns_gpu* g, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K, float* out, int64_t T,
                         int64_t H, int64_t G, int64_t pos0, float scale, int64_t S, float* part) {
    if (S < 0) return ns_fail("ns_mm3s_attend_split: a split count");
    return mm3_attend(g, "ns_mm3s_attend_split", q, kc, vc, sel, K, out, T, H, G, pos0, scale, 1, -1, part, T * G * S * 16 * 130);
}

int ns_mm3s_attend_x_split(ns_gpu* g, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K, float* out, int64_t T,
                           int64_t H, int64_t G, int64_t pos0, float scale, int64_t S, float* part) {
    if (S < 0) return ns_fail("ns_mm3s_attend_x_split: a split count");
    return mm3_attend(g, "ns_mm3s_attend_x_split", q, kc, vc, sel, K, out, T, H, G, pos0, mm3x_scale(scale), 1, -1, part, T * G * S * 16 * 130);
}

int ns_mm3s_attend_block(ns_gpu* g, const float* q, const uint16_t* kc, const uint16_t* vc, float* out, int64_t T, int64_t H, int64_t G, int64_t pos0,
                         int64_t w0, int64_t S, float* part) {
    if (S < 0 || w0 < 0) return ns_fail("ns_mm3s_attend_block: a split count and a first key");
    return mm3_attend(g, "ns_mm3s_attend_block", q, kc, vc, nullptr, 0, out, T, H, G, pos0, 0.08838834764831845f, 0, w0, part, T * G * S * 16 * 130);
}

}  // extern "C"

// ---- tuning knobs (tests and sweeps): read from the environment once, then only changed through ns_attn_tune

namespace {
const char* const TUNE_ENV[NS_TUNE_KNOBS] = {"NS_DEC_WGS", "NS_PREFILL_SPLITS", "NS_PREFILL_WAVES", "NS_MLA_WGS", "NS_PRE_HPW", "NS_PREFILL_BF16", "NS_SCRATCH_MIB"};
std::atomic<int64_t>* tune_table() {
    static std::atomic<int64_t> t[NS_TUNE_KNOBS];
    static const bool once = [] {
        for (int i = 0; i < NS_TUNE_KNOBS; ++i) {
            const char* e = getenv(TUNE_ENV[i]);
            t[i].store(e ? std::max<int64_t>(0, atoll(e)) : 0);
        }
        return true;
    }();
    (void) once;
    return t;
}
}  // namespace

int64_t ns_tune_get(int knob) { return knob >= 0 && knob < NS_TUNE_KNOBS ? tune_table()[knob].load(std::memory_order_relaxed) : 0; }

extern "C" {

int ns_attn_tune(int knob, int64_t value) {
    if (knob < 0 || knob >= NS_TUNE_KNOBS || value < 0) return ns_fail("ns_attn_tune: a knob 0..6 and a value of 0 (the default) or more");
    tune_table()[knob].store(value, std::memory_order_relaxed);
    return 0;
}

}  // extern "C"
