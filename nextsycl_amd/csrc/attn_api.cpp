// attn_api.cpp: the reference engines' attention entry points (ns_q35_*, ns_mg_*, ns_llm_minimaxm3_attend) routed to the
// two kernels of this library: the split-K decode kernel for passes of 1..16 rows, the flash prefill kernel for longer
// ones. Names, arguments and error behaviour follow the reference headers cited in ns_attn.h; zero-row calls return 0
// before anything is checked, as the reference's do (kernels/llm/qwen35/q35.cpp:598).
#include "ns_internal.hpp"
#include "ns_attn.h"

int ns_attn_decode_any(ns_gpu* g, const char* who, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T,
                       int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, int causal, float scale, void* out,
                       float* scratch);
int ns_attn_prompt_any(ns_gpu* g, const char* who, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T,
                       int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, float scale, void* out);
int ns_attn_decode_sel(ns_gpu* g, const char* who, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K,
                       float* out, int64_t T, int64_t Hq, int64_t Hkv, int64_t pos0, float scale, float* scratch, size_t scratch_floats);

namespace {
constexpr int64_t DECODE_ROWS = 16;   // passes up to this many rows take the decode kernel
}

extern "C" {

// ---- prompt form ------------------------------------------------------------------------------------------------------

int ns_mg_attn_prompt_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D) {
    return T > DECODE_ROWS && (D == 128 || D == 256) && Hkv > 0 && Hq > 0 && Hq % Hkv == 0;
}

int ns_mg_attn_prompt(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap,
                      int64_t p0, int64_t win, float* out) {
    if (!ns_mg_attn_prompt_supported(T, Hq, Hkv, D)) return ns_fail("ns_mg_attn_prompt: more than 16 rows, heads of 128 or 256, query heads a multiple of the key heads");
    return ns_attn_prompt_any(g, "ns_mg_attn_prompt", 0, 0, 0, q, Hq * D, kc, vc, T, Hq, Hkv, D, cap, p0, win, 0.0f, out);
}

int ns_q35_attn_prompt_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D) { return ns_mg_attn_prompt_supported(T, Hq, Hkv, D); }

int ns_q35_attn_prompt(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D,
                       int64_t cap, int64_t p0, float* out) {
    if (!ns_q35_attn_prompt_supported(T, Hq, Hkv, D)) return ns_fail("ns_q35_attn_prompt: more than 16 rows, heads of 128 or 256, query heads a multiple of the key heads");
    return ns_attn_prompt_any(g, "ns_q35_attn_prompt", 0, 0, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, 0.0f, out);
}

int ns_q35_attn_prompt_kv(ns_gpu* g, int kt, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv,
                          int64_t D, int64_t cap, int64_t p0, float* out) {
    if (!ns_q35_attn_prompt_supported(T, Hq, Hkv, D)) return ns_fail("ns_q35_attn_prompt_kv: more than 16 rows, heads of 128 or 256, query heads a multiple of the key heads");
    if (kt < 0 || kt > 2) return ns_fail("ns_q35_attn_prompt_kv: a cache form 0 (half), 1 (q8_0) or 2 (q4_0)");
    return ns_attn_prompt_any(g, "ns_q35_attn_prompt_kv", 0, kt, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, 0.0f, out);
}

// ---- the engines' own entry points: decode rows split, prompt rows flash -------------------------------------------------

int64_t ns_q35_attn_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0) {
    return T >= 1 && T <= DECODE_ROWS ? ns_attn_decode_scratch(T, Hq, Hkv, D, p0, 0) : 0;
}

int ns_q35_attn(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D,
                int64_t cap, int64_t p0, float* out, float* scratch) {
    if (T <= 0) return 0;
    if (p0 + T > cap) return ns_fail("ns_q35_attn: past the cache's capacity");
    if (T <= DECODE_ROWS) return ns_attn_decode_any(g, "ns_q35_attn", 0, 0, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, 1, 0.0f, out, scratch);
    return ns_attn_prompt_any(g, "ns_q35_attn", 0, 0, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, 0.0f, out);
}

int64_t ns_mg_attn_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0, int64_t win, int causal) {
    (void) causal;
    return T >= 1 && T <= DECODE_ROWS ? ns_attn_decode_scratch(T, Hq, Hkv, D, p0, win) : 0;
}

int ns_mg_attn(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0,
               int64_t win, int causal, float* out, float* scratch) {
    if (T <= 0) return 0;
    if (T <= DECODE_ROWS) return ns_attn_decode_any(g, "ns_mg_attn", 0, 0, 0, q, Hq * D, kc, vc, T, Hq, Hkv, D, cap, p0, win, causal ? 1 : 0, 0.0f, out, scratch);
    if (!causal) return ns_fail("ns_mg_attn: a block that is not causal has at most 16 rows");
    return ns_attn_prompt_any(g, "ns_mg_attn", 0, 0, 0, q, Hq * D, kc, vc, T, Hq, Hkv, D, cap, p0, win, 0.0f, out);
}

// ---- MiniMax-M3: position-major cache, explicit scale, no scratch argument ------------------------------------------------

int ns_llm_minimaxm3_attend(ns_gpu* g, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K, float* out, int64_t T,
                            int64_t H, int64_t G, int64_t pos0, float scale) {
    if (T <= 0) return 0;
    if (G <= 0 || H % G) return ns_fail("ns_llm_minimaxm3_attend: heads");
    if (!(scale > 0.0f)) return ns_fail("ns_llm_minimaxm3_attend: a positive scale");
    if (sel) return ns_attn_decode_sel(g, "ns_llm_minimaxm3_attend", q, kc, vc, sel, K, out, T, H, G, pos0, scale, g->own_scratch, g->own_scratch_floats);
    const int64_t cap = pos0 + T;
    if (T <= DECODE_ROWS) {
        const int64_t need = ns_attn_decode_scratch(T, H, G, 128, pos0, 0);
        if ((size_t) need > g->own_scratch_floats) return ns_fail("ns_llm_minimaxm3_attend: the pass needs more scratch than the library keeps");
        return ns_attn_decode_any(g, "ns_llm_minimaxm3_attend", 0, 0, 1, q, H * 128, kc, vc, T, H, G, 128, cap, pos0, 0, 1, scale, out, g->own_scratch);
    }
    return ns_attn_prompt_any(g, "ns_llm_minimaxm3_attend", 0, 0, 1, q, H * 128, kc, vc, T, H, G, 128, cap, pos0, 0, scale, out);
}

}  // extern "C"
