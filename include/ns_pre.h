/* ns_pre.h: the step in front of attention on every token - q / k RMS norm, rotary positions, and the KV store - as the
 * reference's entry points (same names, argument order and meaning) plus one fused launch that does all three.
 * All calls are queued on the ns_gpu's compute stream, return 0 or -1 (+ ns_last_error()), allocate nothing. */
#ifndef NS_PRE_H
#define NS_PRE_H
#include <stdint.h>
#include "ns.h"
#ifdef __cplusplus
extern "C" {
#endif

/* kernels/llm/qwen35/q35.h:16-19, q35.cpp:220-254. Per (row t, head h): x = src[t * ss + h * hs .. + D] RMS-normed
 * (weight w [D], eps), then rotate-half rotary positions on its first n_rot features (pairs i, i + n_rot / 2; angle
 * (p0 + t) * theta^(-2 i / n_rot)); into dst[t * ds + h * D]. */
int ns_q35_qk_norm_rope(ns_gpu* g, const float* src, int64_t ss, int64_t hs, float* dst, int64_t ds, int64_t T, int64_t H, int64_t D,
                        const float* w, float eps, int64_t n_rot, float theta, int64_t p0);
/* kernels/llm/qwen35/q35.h:20-24, q35.cpp:350-386. As above, each row at its own positions: pos [T][3] (t, h, w); pair k
 * of the first n_rot turns by one of them as the interleaved sections (s0, s1, s2) choose. */
int ns_q35_qk_norm_rope_pos(ns_gpu* g, const float* src, int64_t ss, int64_t hs, float* dst, int64_t ds, int64_t T, int64_t H, int64_t D,
                            const float* w, float eps, int64_t n_rot, float theta, const int32_t* pos, int64_t s0, int64_t s1, int64_t s2);
/* kernels/llm/qwen35/q35.h:58-60, q35.cpp:256-279. As ns_q35_qk_norm_rope without the norm. */
int ns_q35_rope(ns_gpu* g, const float* src, int64_t ss, int64_t hs, float* dst, int64_t ds, int64_t T, int64_t H, int64_t D, int64_t n_rot,
                float theta, int64_t p0);
/* kernels/llm/ricursive/rc.h:17-21, rc.cpp:148-181. As ns_q35_qk_norm_rope with the rotation over all D features
 * (rope != 0) or none (rope 0). */
int ns_rc_qk_norm_rope(ns_gpu* g, const float* src, int64_t ss, int64_t hs, float* dst, int64_t ds, int64_t T, int64_t H, int64_t D,
                       const float* w, float eps, int rope, float theta, int64_t p0);
/* kernels/llm/museglimmer/mg.h:19-20, mg.cpp:157-190. y[t * ys + h * D ..] = RMS norm of x[t * xs + h * D ..] (weight w,
 * eps), then rotary positions over all D: rope 0 none, 1 adjacent pairs (2i, 2i + 1), 2 halves (i, i + D / 2); angle
 * (p0 + t) * theta^(-2 i / D). y may be x. */
int ns_mg_qk_norm_rope(ns_gpu* g, const float* x, int64_t xs, float* y, int64_t ys, int64_t T, int64_t H, int64_t D, const float* w, float eps,
                       int rope, float theta, int64_t p0);
/* kernels/llm/minimaxm3/mm3.cpp:18-35. In place: rotate-half on the first n_rot of each head of x [T][row] (heads of
 * `head` floats); the angle of pair i is (pos0 + t) multiplied i times by base^(-2 / n_rot). */
int ns_llm_minimaxm3_rope(ns_gpu* g, float* x, int64_t T, int64_t H, int64_t row, int64_t head, int64_t n_rot, int64_t pos0, float base);
/* kernels/llm/minimaxm3/silo/mm3s.h:47-49, moe.cpp:460-501. A decode token's attention after its projections: q [H][HD],
 * k [G][HD], iq [IH][HD], ik [HD] normed (weights qn, kn, iqn, ikn) and rotated in place; k, v, ik stored as half at kc,
 * vc, ic (the token's rows); IH = 0: no indexer. */
int ns_mm3s_attn_post(ns_gpu* g, float* q, float* k, const float* v, float* iq, float* ik, const float* qn, const float* kn, const float* iqn,
                      const float* ikn, uint16_t* kc, uint16_t* vc, uint16_t* ic, int64_t H, int64_t G, int64_t IH, int64_t HD, int64_t n_rot,
                      int64_t pos, float base, float eps);

/* No counterpart in the reference (it runs ns_*_qk_norm_rope twice, then ns_*_kv_store: three launches, k written and
 * read back as float32). One launch: q heads normed and rotated into qo (rows of type qt: 0 float32, 1 half, 2
 * bfloat16; qos elements a row), k heads normed, rotated and written straight into the cache in its row form kt (0 half,
 * 1 q8_0, 2 q4_0, 3 bfloat16), v heads written into theirs; caches head-major [Hkv][cap][row], slot p0 + t (ring: % cap).
 * rope: 1 = ns_q35_qk_norm_rope's (rotate-half over n_rot), 2 / 3 = ns_mg_qk_norm_rope's rope 1 / 2 (n_rot ignored).
 * Bit for bit what the separate calls give (same arithmetic). D 64, 128 or 256. */
int ns_attn_pre_store(ns_gpu* g, int rope, int qt, int kt, int ring, const float* q, int64_t qss, int64_t qhs, void* qo, int64_t qos,
                      const float* k, int64_t kss, int64_t khs, const float* v, int64_t vss, const float* qw, const float* kw, float eps,
                      int64_t n_rot, float theta, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, void* kc, void* vc);

#ifdef __cplusplus
}
#endif
#endif
