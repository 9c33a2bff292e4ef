/* oracle.c - TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C CPU restatement of the arithmetic of nextsycl's LLM attention path, used only as the checker in tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg. Nothing in the shipped library links, loads or calls it.
 * Every function cites the reference file:line it follows (paths relative to the reference tree).
 *
 * Two kinds of functions live here:
 *   - "order" restatements: float32, the same operation order as the reference's exact (vector-unit) kernels
 *     (streams of keys, split/merge with exp) - orc_attn_exact, orc_mla_decode, orc_mm3_attend, orc_glm_mla_attend - and
 *     of the norm + rotary-position step in front of attention - orc_q35_norm_rope, orc_mg_norm_rope, orc_mm3_norm_rope_row;
 *   - float64 closed forms softmax(q k^T s + mask) v on the very same stored (f16 / q8_0 / q4_0 / bf16) values -
 *     orc_attn_f64, orc_mla_f64: the tolerance arm (max-abs 2e-3, relative L2 1e-3 for f16/bf16 outputs).
 * Integer/byte work (cache rows, q8_0 / q4_0 packing, dequant, split arithmetic) is restated exactly and compared
 * bit for bit.
 *
 * What pins each function (see tests/test_oracle_*.py): closed forms evaluated independently in numpy float64,
 * hand-derived known answers for the quantizers (ggml's quantize_row_q8_0_ref / q4_0_ref rules), numpy.float16 for
 * the half conversions over every bit pattern, partition invariance of the split/merge, brute force on tiny
 * shapes, and for the rotary positions a float64 complex-rotation statement in numpy plus the rotation's invariants
 * (position 0 is the identity, a pair's norm is kept, angles add). The reference ships no golden vectors for this path.
 *
 * Parity unpinned: none of the functions below.
 *
 * Build: gcc -O3 -march=native -fopenmp -ffp-contract=off -shared -fPIC oracle.c -o liboracle.so -lm
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------------------ conversions */

/* float -> IEEE half, round to nearest even (what sycl::half(float) does; kernels/llm/qwen35/q35.cpp:584) */
ORC_API uint16_t orc_f2h(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint16_t s = (uint16_t) ((x >> 16) & 0x8000u);
    const uint32_t a = x & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t) (s | 0x7e00u);
    if (a >= 0x477ff000u) return (uint16_t) (s | 0x7c00u);
    if (a < 0x33000001u) return s;
    const int e = (int) (a >> 23) - 127;
    const uint32_t m = (a & 0x7fffffu) | 0x800000u;
    const int shift = e < -14 ? 13 + (-14 - e) : 13;
    uint32_t hm = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (hm & 1u))) ++hm;
    if (e < -14) return (uint16_t) (s | hm);
    return (uint16_t) (s | (uint16_t) ((((uint32_t) (e + 15)) << 10) + (hm - 0x400u)));
}

ORC_API float orc_h2f(uint16_t h) {
    const uint32_t s = ((uint32_t) h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu, x;
    if (e == 0) {
        if (m == 0) {
            x = s;
        } else {
            int k = 0;
            while (!(m & 0x400u)) { m <<= 1; ++k; }
            x = s | ((uint32_t) (113 - k) << 23) | ((m & 0x3ffu) << 13);
        }
    } else if (e == 31) {
        x = s | 0x7f800000u | (m << 13);
    } else {
        x = s | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

/* float -> bfloat16, round to nearest even (the build's own bf16 caches; the reference has no bf16) */
ORC_API uint16_t orc_f2bf(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t) ((x >> 16) | 0x40u);
    x += 0x7fffu + ((x >> 16) & 1u);
    return (uint16_t) (x >> 16);
}

ORC_API float orc_bf2f(uint16_t b) {
    const uint32_t x = (uint32_t) b << 16;
    float f;
    memcpy(&f, &x, 4);
    return f;
}

ORC_API void orc_f2h_n(const float* x, uint16_t* y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = orc_f2h(x[i]); }
ORC_API void orc_h2f_n(const uint16_t* x, float* y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = orc_h2f(x[i]); }
ORC_API void orc_f2bf_n(const float* x, uint16_t* y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = orc_f2bf(x[i]); }
ORC_API void orc_bf2f_n(const uint16_t* x, float* y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = orc_bf2f(x[i]); }

/* ------------------------------------------------------------------------------------------------ seeded inputs */

/* xorshift64* as the reference's own kernel checks draw their inputs (llm/deepseek2/src/tools.rs:14-23): the top 24
 * bits of the product as a uniform in [0, 1) */
static inline uint32_t xs_next24(uint64_t* s) {
    *s ^= *s >> 12;
    *s ^= *s << 25;
    *s ^= *s >> 27;
    return (uint32_t) ((*s * 0x2545F4914F6CDD1DULL) >> 40);
}

ORC_API void orc_uniform_f32(uint64_t seed, float* out, int64_t n) {
    uint64_t s = seed;
    for (int64_t i = 0; i < n; ++i) out[i] = (float) xs_next24(&s) / 16777216.0f;
}

/* N(0, sigma): two uniforms -> Box-Muller in float64 (u1 = (k1 + 1) / 2^24 in (0, 1], u2 = k2 / 2^24), both branches
 * used (cos for element 2i, sin for 2i + 1), scaled by sigma, rounded to float32 */
ORC_API void orc_randn_f32(uint64_t seed, double sigma, float* out, int64_t n) {
    uint64_t s = seed;
    for (int64_t i = 0; i < n; i += 2) {
        const double u1 = ((double) xs_next24(&s) + 1.0) / 16777216.0, u2 = (double) xs_next24(&s) / 16777216.0;
        const double r = sqrt(-2.0 * log(u1)), a = 6.283185307179586476925286766559 * u2;
        out[i] = (float) (sigma * r * cos(a));
        if (i + 1 < n) out[i + 1] = (float) (sigma * r * sin(a));
    }
}

/* ------------------------------------------------------------------------------------------------ cache rows */

/* kt: 0 half [D], 1 q8_0 ([D int8][D/32 half]), 2 q4_0 ([D/2 bytes][D/32 half]) - llm/qwen35/src/engine.rs:44-60,
 * kernels/llm/qwen35/silo/attn.cpp:43-46; 3 bfloat16 [D] (the build's own addition) */
ORC_API int64_t orc_kv_row_bytes(int kt, int64_t D) {
    switch (kt) {
        case 0: return 2 * D;
        case 1: return D + D / 32 * 2;
        case 2: return D / 2 + D / 32 * 2;
        case 3: return 2 * D;
        default: return -1;
    }
}

static inline uint16_t ld16(const uint8_t* p) { uint16_t v; memcpy(&v, p, 2); return v; }
static inline void st16(uint8_t* p, uint16_t v) { memcpy(p, &v, 2); }

/* value i of a cache row of form kt as float32 - kernels/llm/qwen35/q35.cpp:19-25 (D generalised from 256) */
ORC_API float orc_kv_value(const uint8_t* row, int kt, int64_t D, int64_t i) {
    if (kt == 0) return orc_h2f(ld16(row + 2 * i));
    if (kt == 3) return orc_bf2f(ld16(row + 2 * i));
    const int64_t b = i / 32, j = i % 32;
    if (kt == 1) return (float) (int8_t) row[i] * orc_h2f(ld16(row + D + 2 * b));
    const uint8_t w = row[b * 16 + (j & 15)];
    return (float) ((int) (j < 16 ? w & 15 : w >> 4) - 8) * orc_h2f(ld16(row + D / 2 + 2 * b));
}

/* the same value as the XMX kernels stage it: rounded to half before the product -
 * kernels/llm/qwen35/silo/attn.cpp:56-60,70-76 */
ORC_API uint16_t orc_kv_value_h(const uint8_t* row, int kt, int64_t D, int64_t i) {
    if (kt == 0) return ld16(row + 2 * i);
    return orc_f2h(orc_kv_value(row, kt, D, i));
}
/* as a float: the staged 16-bit value widened again (a bfloat16 cache's values are staged as they are) */
static inline float kv_staged(const uint8_t* row, int kt, int64_t D, int64_t i) {
    if (kt == 3) return orc_bf2f(ld16(row + 2 * i));
    return orc_h2f(orc_kv_value_h(row, kt, D, i));
}

/* rows dequantized to float32: out [n][D] from rows `stride` bytes apart */
ORC_API void orc_kv_dequant(const uint8_t* rows, int kt, int64_t D, int64_t n, int64_t stride, float* out) {
    for (int64_t r = 0; r < n; ++r)
        for (int64_t i = 0; i < D; ++i) out[r * D + i] = orc_kv_value(rows + r * stride, kt, D, i);
}

/* f32 k, v rows -> half caches [Hkv][cap][D] at positions p0.. - kernels/llm/qwen35/q35.cpp:573-588; ring != 0: slot
 * (p0 + t) % cap - kernels/llm/museglimmer/mg.cpp:192-206; kt 3 stores bfloat16 instead. -1: past the capacity */
ORC_API int orc_kv_store(int kt, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D, int64_t cap,
                         int64_t p0, int ring, uint8_t* kc, uint8_t* vc) {
    if (T <= 0) return 0;
    if (ring ? T > cap : p0 + T > cap) return -1;
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < Hkv; ++h)
            for (int64_t d = 0; d < D; ++d) {
                const int64_t slot = ring ? (p0 + t) % cap : p0 + t, at = ((h * cap + slot) * D + d) * 2;
                const float kf = k[t * ks + h * D + d], vf = v[t * vs + h * D + d];
                st16(kc + at, kt == 3 ? orc_f2bf(kf) : orc_f2h(kf));
                st16(vc + at, kt == 3 ? orc_f2bf(vf) : orc_f2h(vf));
            }
    return 0;
}

/* one block of 32 as q8_0: amax / 127, the reciprocal multiplied, round half away from zero, the scale stored as half
 * but not used for quantizing - kernels/llm/qwen35/q35.cpp:301-306 (= ggml quantize_row_q8_0_ref) */
static void q8_0_block(const float* x, uint8_t* qs, uint8_t* scale) {
    float amax = 0.0f;
    for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(x[j]));
    const float d = amax / 127.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
    for (int j = 0; j < 32; ++j) qs[j] = (uint8_t) (int8_t) roundf(x[j] * id);
    st16(scale, orc_f2h(d));
}

/* one block of 32 as q4_0: the value of the largest magnitude (the first of a tie) / -8; byte j = value j low nibble,
 * value j + 16 high - kernels/llm/qwen35/q35.cpp:307-321 (= ggml quantize_row_q4_0_ref) */
static void q4_0_block(const float* x, uint8_t* qs, uint8_t* scale) {
    float m = 0.0f, am = 0.0f;
    for (int j = 0; j < 32; ++j)
        if (fabsf(x[j]) > am) { am = fabsf(x[j]); m = x[j]; }
    const float d = m / -8.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
    for (int j = 0; j < 16; ++j) {
        int lo = (int) (x[j] * id + 8.5f), hi = (int) (x[j + 16] * id + 8.5f);
        if (lo > 15) lo = 15;
        if (hi > 15) hi = 15;
        qs[j] = (uint8_t) (lo | (hi << 4));
    }
    st16(scale, orc_f2h(d));
}

/* f32 k, v rows -> q8_0 (kt 1) / q4_0 (kt 2) caches [Hkv][cap][row bytes], the scales behind the row's values -
 * kernels/llm/qwen35/q35.cpp:281-326 (the reference accepts D = 256 only; any multiple of 32 here) */
ORC_API int orc_kv_store_q(int kt, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D, int64_t cap,
                           int64_t p0, uint8_t* kc, uint8_t* vc) {
    if (T <= 0) return 0;
    if ((kt != 1 && kt != 2) || D % 32) return -1;
    if (p0 + T > cap) return -1;
    const int64_t rb = orc_kv_row_bytes(kt, D), nb = D / 32;
    for (int isv = 0; isv < 2; ++isv)
        for (int64_t t = 0; t < T; ++t)
            for (int64_t h = 0; h < Hkv; ++h)
                for (int64_t b = 0; b < nb; ++b) {
                    const float* x = (isv ? v + t * vs : k + t * ks) + h * D + b * 32;
                    uint8_t* row = (isv ? vc : kc) + (h * cap + p0 + t) * rb;
                    if (kt == 1) q8_0_block(x, row + b * 32, row + D + 2 * b);
                    else q4_0_block(x, row + b * 16, row + D / 2 + 2 * b);
                }
    return 0;
}

/* normalized 32-point Walsh-Hadamard transform of each block of 32 - kernels/llm/qwen35/q35.cpp:328-348 */
ORC_API void orc_fwht32(float* x, int64_t rows, int64_t n, int64_t stride) {
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t b = 0; b < n / 32; ++b) {
            float* p = x + r * stride + b * 32;
            float v[32];
            for (int i = 0; i < 32; ++i) v[i] = p[i];
            for (int o = 1; o < 32; o <<= 1)
                for (int i = 0; i < 32; ++i)
                    if (!(i & o)) {
                        const float a = v[i], c = v[i + o];
                        v[i] = a + c;
                        v[i + o] = a - c;
                    }
            for (int i = 0; i < 32; ++i) p[i] = v[i] * 0.17677669529663687f;
        }
}

/* GLM-5.3's q8 latent row [L/32 half scales][L int8]: the scale rounded to half BEFORE it divides, clamp to +-127 -
 * kernels/llm/glm5next/glm.cpp:1282-1299 */
ORC_API void orc_glm_to_q8row(const float* x, uint8_t* y, int64_t n, int64_t L) {
    const int64_t nb = L / 32, rb = nb * 2 + L;
    for (int64_t r = 0; r < n; ++r)
        for (int64_t b = 0; b < nb; ++b) {
            const float* xb = x + r * L + b * 32;
            float amax = 0.0f;
            for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(xb[j]));
            const uint16_t dh = orc_f2h(amax / 127.0f);
            const float d = orc_h2f(dh), inv = d > 0.0f ? 1.0f / d : 0.0f;
            st16(y + r * rb + 2 * b, dh);
            for (int j = 0; j < 32; ++j) {
                float q = roundf(xb[j] * inv);
                q = fminf(127.0f, fmaxf(-127.0f, q));
                y[r * rb + nb * 2 + b * 32 + j] = (uint8_t) (int8_t) q;
            }
        }
}

/* ------------------------------------------------------------------------------------------------ split rules */

static inline int64_t imax(int64_t a, int64_t b) { return a > b ? a : b; }
static inline int64_t imin(int64_t a, int64_t b) { return a < b ? a : b; }

/* the exact kernels' keys a split - kernels/llm/qwen35/q35.cpp:34-42 (decode rows only: S == 1) */
ORC_API int64_t orc_q35_split_keys(int64_t S, int64_t kv, int64_t Hkv) {
    if (S != 1) return kv;
    const int64_t want = (kv * Hkv + 511) / 512;
    return imax(32, (want + 31) / 32 * 32);
}
ORC_API int64_t orc_q35_splits(int64_t S, int64_t kv, int64_t Hkv) {
    const int64_t kb = orc_q35_split_keys(S, kv, Hkv);
    return kv > kb ? (kv + kb - 1) / kb : 1;
}
/* kernels/llm/museglimmer/mg.cpp:23-37 (S <= 16: a verify pass's rows split too; groups = Hq / 4) */
ORC_API int64_t orc_mg_split_keys(int64_t S, int64_t kv, int64_t groups) {
    if (S > 16) return kv;
    const int64_t want = (kv * groups + 511) / 512;
    return imax(32, (want + 31) / 32 * 32);
}
ORC_API int64_t orc_mg_seen(int64_t S, int64_t p0, int64_t win, int causal) {
    const int64_t end = p0 + S;
    if (win <= 0) return end;
    return causal ? imin(end, win) : end - imax(0, p0 + 1 - win);
}
ORC_API int64_t orc_mg_splits(int64_t S, int64_t kv, int64_t groups) {
    const int64_t kb = orc_mg_split_keys(S, kv, groups);
    return kv > kb ? (kv + kb - 1) / kb : 1;
}
/* the XMX decode kernels' keys a split: ~512 work-groups, multiples of 64 - kernels/llm/qwen35/silo/attn.cpp:321-331 */
ORC_API int64_t orc_dec_split(int64_t kv, int64_t Hkv) {
    const int64_t want = (kv * Hkv + 511) / 512;
    return imax(64, (want + 63) / 64 * 64);
}
ORC_API int64_t orc_dec_splits(int64_t kv, int64_t Hkv) { return (kv + orc_dec_split(kv, Hkv) - 1) / orc_dec_split(kv, Hkv); }
/* floats of scratch the reference's decode asks for - kernels/llm/qwen35/silo/attn.cpp:406-410 */
ORC_API int64_t orc_q35_attn_decode_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0) {
    int64_t ns = 1;
    for (int64_t r = 0; r < T; ++r) ns = imax(ns, orc_dec_splits(p0 + r + 1, Hkv));
    return ns > 1 ? T * Hq * ns * (D + 2) : 0;
}

/* ------------------------------------------------------------------------------------------------ GQA attention */

/* address of the cache row of key head hk, slot: head-major [Hkv][cap][row] when pm == 0
 * (kernels/llm/qwen35/q35.h:55-57), position-major [pos][Hkv][row] when pm != 0 (kernels/llm/minimaxm3/mm3.h:33-36) */
static inline const uint8_t* kv_row_at(const uint8_t* c, int pm, int64_t Hkv, int64_t cap, int64_t rb, int64_t hk, int64_t slot) {
    return pm ? c + (slot * Hkv + hk) * rb : c + (hk * cap + slot) * rb;
}

/* One (row, query head) of the reference's exact kernel, its operation order kept: NSTREAM (4) streams take the
 * split's keys in turn (stream k: j0 + k, j0 + k + 4, ...), each an online softmax with exp in float32; the streams
 * merged with exp(m_k - mx); the splits merged the same way - kernels/llm/museglimmer/mg.cpp:40-149 (D 128),
 * kernels/llm/qwen35/q35.cpp:44-148 (D 256). A key's score: each of 16 lanes sums its D/16 products in order, the 16
 * lane sums added as a butterfly (the device's reduce_over_group order is not specified; any order is within float32
 * reassociation error). */
static void attn_exact_row(const float* qrow, const uint8_t* kc, const uint8_t* vc, int kt, int pm, int64_t Hkv, int64_t hk, int64_t D,
                           int64_t cap, int64_t first, int64_t end, int64_t KB, int64_t ns, float* out) {
    enum { NS = 4, LANES = 16 };
    const int64_t rb = orc_kv_row_bytes(kt, D), DL = D / LANES, n = end - first;
    const float scale = 1.0f / sqrtf((float) D);
    float* qv = (float*) malloc(sizeof(float) * D);
    float* kf = (float*) malloc(sizeof(float) * D);
    float* acc = (float*) malloc(sizeof(float) * NS * D);
    float* pa = (float*) malloc(sizeof(float) * ns * (D + 2));
    for (int64_t d = 0; d < D; ++d) qv[d] = qrow[d] * scale;
    for (int64_t sp = 0; sp < ns; ++sp) {
        const int64_t j0 = first + sp * (ns > 1 ? KB : n), j1 = imin(end, ns > 1 ? first + (sp + 1) * KB : end);
        float m[NS], l[NS];
        for (int k = 0; k < NS; ++k) {
            m[k] = -INFINITY;
            l[k] = 0.0f;
            for (int64_t d = 0; d < D; ++d) acc[k * D + d] = 0.0f;
        }
        for (int k = 0; k < NS; ++k)
            for (int64_t j = j0 + k; j < j1; j += NS) {
                const int64_t slot = j % cap;
                const uint8_t* kr = kv_row_at(kc, pm, Hkv, cap, rb, hk, slot);
                const uint8_t* vr = kv_row_at(vc, pm, Hkv, cap, rb, hk, slot);
                float lane[LANES];
                for (int ln = 0; ln < LANES; ++ln) {
                    float dsum = 0.0f;
                    for (int64_t i = 0; i < DL; ++i) dsum += qv[ln * DL + i] * orc_kv_value(kr, kt, D, ln * DL + i);
                    lane[ln] = dsum;
                }
                for (int o = LANES / 2; o > 0; o >>= 1)
                    for (int ln = 0; ln < o; ++ln) lane[ln] += lane[ln + o];
                const float sc = lane[0];
                const float mn = fmaxf(m[k], sc);
                const float c = expf(m[k] - mn), e = expf(sc - mn);
                for (int64_t d = 0; d < D; ++d) kf[d] = orc_kv_value(vr, kt, D, d);
                for (int64_t d = 0; d < D; ++d) acc[k * D + d] = acc[k * D + d] * c + e * kf[d];
                l[k] = l[k] * c + e;
                m[k] = mn;
            }
        float mx = -INFINITY;
        for (int k = 0; k < NS; ++k) mx = fmaxf(mx, m[k]);
        float* p = pa + sp * (D + 2);
        for (int64_t d = 0; d < D; ++d) {
            float L = 0.0f, A = 0.0f;
            if (mx != -INFINITY)
                for (int k = 0; k < NS; ++k) {
                    const float e = expf(m[k] - mx);
                    L += l[k] * e;
                    A += acc[k * D + d] * e;
                }
            p[d] = A;
            p[D + 1] = L;
        }
        p[D] = mx;
    }
    if (ns == 1) {
        for (int64_t d = 0; d < D; ++d) out[d] = pa[D + 1] > 0.0f ? pa[d] / pa[D + 1] : 0.0f;
    } else {
        float mx = -INFINITY;
        for (int64_t k = 0; k < ns; ++k) mx = fmaxf(mx, pa[k * (D + 2) + D]);
        for (int64_t d = 0; d < D; ++d) {
            float L = 0.0f, A = 0.0f;
            if (mx != -INFINITY)
                for (int64_t k = 0; k < ns; ++k) {
                    const float e = expf(pa[k * (D + 2) + D] - mx);
                    L += pa[k * (D + 2) + D + 1] * e;
                    A += pa[k * (D + 2) + d] * e;
                }
            out[d] = L > 0.0f ? A / L : 0.0f;
        }
    }
    free(qv);
    free(kf);
    free(acc);
    free(pa);
}

/* The reference's exact attention for a pass of T rows at p0.. (float32 q [T][Hq*D] rows qs apart, out [T][Hq*D]):
 * row r sees keys max(0, pos + 1 - win) .. pos (causal) or .. p0 + T - 1 (not causal); slot = position % cap. The
 * split rule: decode rows (T <= 16, causal) each split as their own one-row pass would be, prompt rows one split -
 * kernels/llm/museglimmer/mg.cpp:208-253; the caller passes the rule's `groups` (mg: Hq / 4). split_single_only != 0
 * is the qwen35 engine's rule, where only a one-row pass splits and `groups` is Hkv -
 * kernels/llm/qwen35/q35.cpp:34-42,590-612.
 * pm: cache layout (0 head-major, 1 position-major). */
ORC_API int orc_attn_exact(const float* q, int64_t qs, const uint8_t* kc, const uint8_t* vc, int kt, int pm, int64_t T, int64_t Hq, int64_t Hkv,
                           int64_t D, int64_t cap, int64_t p0, int64_t win, int causal, int64_t groups, int split_single_only, float* out) {
    if (T <= 0) return 0;
    if (Hkv <= 0 || Hq % Hkv || D % 16 || orc_kv_row_bytes(kt, D) < 0) return -1;
    const int64_t per = Hq / Hkv;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t r = 0; r < T; ++r)
        for (int64_t hq = 0; hq < Hq; ++hq) {
            const int64_t pos = p0 + r, end = causal ? pos + 1 : p0 + T, first = win > 0 ? imax(0, pos + 1 - win) : 0;
            int64_t KB = end - first, ns = 1;
            const int decode_rows = split_single_only ? T == 1 : (T <= 16 && causal);
            if (decode_rows) {
                const int64_t kv = end - first;
                KB = orc_mg_split_keys(1, kv, groups);
                ns = kv > KB ? (kv + KB - 1) / KB : 1;
            }
            attn_exact_row(q + r * qs + hq * D, kc, vc, kt, pm, Hkv, hq / per, D, cap, first, end, KB, ns, out + (r * Hq + hq) * D);
        }
    return 0;
}

/* The closed form in float64 on the stored values: out[r][hq][:] = sum_j softmax_j(scale q.k_j) v_j over the keys
 * the row sees; no key visible -> 0. q is float32 (the caller rounds it to f16 / bf16 first when the config says so).
 * scale <= 0: 1 / sqrt(D). */
static int attn_f64_impl(const float* q, int64_t qs, const uint8_t* kc, const uint8_t* vc, int kt, int pm, int64_t T, int64_t Hq, int64_t Hkv,
                         int64_t D, int64_t cap, int64_t p0, int64_t win, int causal, int64_t kfirst, double scale, double* out) {
    if (T <= 0) return 0;
    if (Hkv <= 0 || Hq % Hkv || orc_kv_row_bytes(kt, D) < 0) return -1;
    const int64_t per = Hq / Hkv, rb = orc_kv_row_bytes(kt, D);
    const double sc = scale > 0.0 ? scale : 1.0 / sqrt((double) D);
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t r = 0; r < T; ++r)
        for (int64_t hq = 0; hq < Hq; ++hq) {
            const int64_t pos = p0 + r, end = causal ? pos + 1 : p0 + T, first = kfirst >= 0 ? kfirst : win > 0 ? imax(0, pos + 1 - win) : 0, hk = hq / per;
            const int64_t n = end - first;
            double* o = out + (r * Hq + hq) * D;
            for (int64_t d = 0; d < D; ++d) o[d] = 0.0;
            if (n <= 0) continue;
            double* s = (double*) malloc(sizeof(double) * n);
            const float* qr = q + r * qs + hq * D;
            double mx = -INFINITY;
            for (int64_t j = first; j < end; ++j) {
                const uint8_t* kr = kv_row_at(kc, pm, Hkv, cap, rb, hk, j % cap);
                double a = 0.0;
                for (int64_t d = 0; d < D; ++d) a += (double) qr[d] * (double) orc_kv_value(kr, kt, D, d);
                s[j - first] = a * sc;
                if (s[j - first] > mx) mx = s[j - first];
            }
            double l = 0.0;
            for (int64_t j = first; j < end; ++j) {
                const double e = exp(s[j - first] - mx);
                l += e;
                const uint8_t* vr = kv_row_at(vc, pm, Hkv, cap, rb, hk, j % cap);
                for (int64_t d = 0; d < D; ++d) o[d] += e * (double) orc_kv_value(vr, kt, D, d);
            }
            for (int64_t d = 0; d < D; ++d) o[d] /= l;
            free(s);
        }
    return 0;
}
ORC_API int orc_attn_f64(const float* q, int64_t qs, const uint8_t* kc, const uint8_t* vc, int kt, int pm, int64_t T, int64_t Hq, int64_t Hkv,
                         int64_t D, int64_t cap, int64_t p0, int64_t win, int causal, double scale, double* out) {
    return attn_f64_impl(q, qs, kc, vc, kt, pm, T, Hq, Hkv, D, cap, p0, win, causal, -1, scale, out);
}
/* the same closed form for a draft block whose rows all start at one key: every row sees kfirst .. p0 + T - 1 (not
 * causal) - kernels/llm/minimaxm3/silo/attnx.cpp:36,60,86 (`pos = pos0 + T - 1`, `total = pos + 1 - w0`, `j0 = c0 + w0`) */
ORC_API int orc_attn_f64_block(const float* q, int64_t qs, const uint8_t* kc, const uint8_t* vc, int kt, int pm, int64_t T, int64_t Hq, int64_t Hkv,
                               int64_t D, int64_t cap, int64_t p0, int64_t kfirst, double scale, double* out) {
    if (kfirst < 0 || kfirst > p0) return -1;
    return attn_f64_impl(q, qs, kc, vc, kt, pm, T, Hq, Hkv, D, cap, p0, 0, 0, kfirst, scale, out);
}

/* The weights one row's heads give every key, reduced over the heads and ADDED to out [n] - kernels/llm/qwen35/q35.cpp:464-506:
 * score(h, j) = (sum_i q[h][i] k_j[i], i ascending, float32) / sqrt(D); per head m = max_j, z = sum_j exp(score - m); per key
 * acc = sum_h p / Hq (mode 0, heads ascending) or max_h p (mode 1), p = exp(score - m) / z. The reference's per-head
 * reductions run over a work-group in an order SYCL leaves open; here the sum over j is ascending. */
ORC_API int orc_attn_probs(int kt, const float* q, const uint8_t* kc, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t n, int mode,
                           float* out) {
    if (n <= 0) return 0;
    if (n > cap || Hkv <= 0 || Hq % Hkv || orc_kv_row_bytes(kt, D) < 0) return -1;
    const int64_t G = Hq / Hkv, rb = orc_kv_row_bytes(kt, D);
    const float scale = 1.0f / sqrtf((float) D);
    float* sc = (float*) malloc(sizeof(float) * (size_t) (Hq * n));
    float* mz = (float*) malloc(sizeof(float) * (size_t) (2 * Hq));
#pragma omp parallel for schedule(static)
    for (int64_t h = 0; h < Hq; ++h) {
        float m = -INFINITY;
        for (int64_t j = 0; j < n; ++j) {
            const uint8_t* row = kc + ((h / G) * cap + j) * rb;
            float a = 0.0f;
            for (int64_t i = 0; i < D; ++i) a += q[h * D + i] * orc_kv_value(row, kt, D, i);
            sc[h * n + j] = a * scale;
            m = fmaxf(m, sc[h * n + j]);
        }
        float z = 0.0f;
        for (int64_t j = 0; j < n; ++j) z += expf(sc[h * n + j] - m);
        mz[2 * h] = m;
        mz[2 * h + 1] = z;
    }
    for (int64_t j = 0; j < n; ++j) {
        float acc = 0.0f;
        for (int64_t h = 0; h < Hq; ++h) {
            const float p = expf(sc[h * n + j] - mz[2 * h]) / mz[2 * h + 1];
            acc = mode == 1 ? fmaxf(acc, p) : acc + p / (float) Hq;
        }
        out[j] += acc;
    }
    free(sc);
    free(mz);
    return 0;
}

/* The rounding model of the reference's XMX flash kernels (kernels/llm/qwen35/silo/attn.cpp:105-313; D 128:
 * kernels/llm/museglimmer/silo/attn.cpp:56-267): q scaled by 1/sqrt(D) log2(e) in float32 and rounded to half; scores
 * float32 sums of half x half products, the two halves of D summed apart and then added (:188-201,213); chunks of 16
 * keys at absolute multiples of 16; base-2 online softmax with c = 1 when the new maximum is -inf (:219-224); the sum
 * of the unrounded weights into l, the weights rounded to half for the value product (:225-233); the key splits of
 * `kbs` keys at absolute positions (0: one split), merged with exp2 (:351-369). Cache values rounded to half as staged
 * (:56-60). The build's GPU kernels follow this model (half operands, float32 accumulation and softmax), not its
 * instruction order. */
ORC_API int orc_attn_flash_model(const float* q, int64_t qs, const uint8_t* kc, const uint8_t* vc, int kt, int pm, int64_t T, int64_t Hq,
                                 int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, int64_t kbs, float* out) {
    if (T <= 0) return 0;
    if (Hkv <= 0 || Hq % Hkv || D % 2 || orc_kv_row_bytes(kt, D) < 0) return -1;
    enum { CH = 16 };
    const int64_t per = Hq / Hkv, rb = orc_kv_row_bytes(kt, D);
    const float qscale = 1.0f / sqrtf((float) D) * 1.4426950408889634f;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t r = 0; r < T; ++r)
        for (int64_t hq = 0; hq < Hq; ++hq) {
            const int64_t pos = p0 + r, end = pos + 1, first = win > 0 ? imax(0, pos + 1 - win) : 0, hk = hq / per;
            const int64_t KB = kbs > 0 ? kbs : end, sp0 = first / KB, ns = (end - 1) / KB - sp0 + 1;
            float* qh = (float*) malloc(sizeof(float) * D);
            float* O = (float*) malloc(sizeof(float) * D);
            float* pa = (float*) malloc(sizeof(float) * ns * (D + 2));
            for (int64_t d = 0; d < D; ++d) qh[d] = orc_h2f(orc_f2h(q[r * qs + hq * D + d] * qscale));
            for (int64_t sp = 0; sp < ns; ++sp) {
                const int64_t jbeg = imax(first, (sp0 + sp) * KB), jend = imin(end, (sp0 + sp + 1) * KB);
                float m = -INFINITY, l = 0.0f;
                for (int64_t d = 0; d < D; ++d) O[d] = 0.0f;
                for (int64_t j0 = jbeg / CH * CH; j0 < jend; j0 += CH) {
                    float s[CH], p[CH], mx = -INFINITY;
                    for (int n = 0; n < CH; ++n) {
                        const int64_t j = j0 + n;
                        s[n] = -INFINITY;
                        if (j > pos || j < first || j < jbeg || j >= jend) continue;
                        const uint8_t* kr = kv_row_at(kc, pm, Hkv, cap, rb, hk, j % cap);
                        float a0 = 0.0f, a1 = 0.0f;
                        for (int64_t d = 0; d < D / 2; ++d) a0 += qh[d] * kv_staged(kr, kt, D, d);
                        for (int64_t d = D / 2; d < D; ++d) a1 += qh[d] * kv_staged(kr, kt, D, d);
                        s[n] = a0 + a1;
                        mx = fmaxf(mx, s[n]);
                    }
                    const float mn = fmaxf(m, mx);
                    const float c = mn == -INFINITY ? 1.0f : exp2f(m - mn);
                    float sum = 0.0f;
                    for (int n = 0; n < CH; ++n) {
                        const float pv = s[n] == -INFINITY ? 0.0f : exp2f(s[n] - mn);
                        sum += pv;
                        p[n] = orc_h2f(orc_f2h(pv));
                    }
                    m = mn;
                    l = l * c + sum;
                    for (int64_t d = 0; d < D; ++d) O[d] *= c;
                    for (int n = 0; n < CH; ++n) {
                        const int64_t j = j0 + n;
                        if (p[n] == 0.0f || j >= jend || j < jbeg) continue;
                        const uint8_t* vr = kv_row_at(vc, pm, Hkv, cap, rb, hk, j % cap);
                        for (int64_t d = 0; d < D; ++d) O[d] += p[n] * kv_staged(vr, kt, D, d);
                    }
                }
                float* pp = pa + sp * (D + 2);
                for (int64_t d = 0; d < D; ++d) pp[d] = O[d];
                pp[D] = m;
                pp[D + 1] = l;
            }
            float* o = out + (r * Hq + hq) * D;
            if (ns == 1) {
                for (int64_t d = 0; d < D; ++d) o[d] = pa[D + 1] > 0.0f ? pa[d] / pa[D + 1] : 0.0f;
            } else {
                float mx = -INFINITY;
                for (int64_t k = 0; k < ns; ++k) mx = fmaxf(mx, pa[k * (D + 2) + D]);
                for (int64_t d = 0; d < D; ++d) {
                    float Ls = 0.0f, A = 0.0f;
                    if (mx != -INFINITY)
                        for (int64_t k = 0; k < ns; ++k) {
                            const float e = exp2f(pa[k * (D + 2) + D] - mx);
                            Ls += pa[k * (D + 2) + D + 1] * e;
                            A += pa[k * (D + 2) + d] * e;
                        }
                    o[d] = Ls > 0.0f ? A / Ls : 0.0f;
                }
            }
            free(qh);
            free(O);
            free(pa);
        }
    return 0;
}

/* MiniMax-M3's exact GQA over a position-major half cache [pos][G][128], explicit scale, chunks of 2048 keys with a
 * chunk-wide maximum, the values summed in key order - kernels/llm/minimaxm3/mm3.cpp:118-190. sel == NULL: dense
 * (keys 0 .. pos); else sel [T][G][K] names K blocks of 128 keys a (row, key head) (-1: none), the keys of a listed block
 * past the row's position dropped (:143-157). */
ORC_API int orc_mm3_attend_sel(const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K, float* out, int64_t T,
                               int64_t H, int64_t G, int64_t pos0, float scale) {
    enum { BLK = 128, CHK = 2048 };
    if (G <= 0 || H % G) return -1;
    const int64_t per = H / G;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t t = 0; t < T; ++t)
        for (int64_t hq = 0; hq < H; ++hq) {
            const int64_t gi = hq / per, pos = pos0 + t, total = sel ? K * BLK : pos + 1;
            const float* qr = q + (t * H + hq) * BLK;
            float sc[CHK], acc[BLK], m = -INFINITY, l = 0.0f;
            int64_t jj[CHK];
            for (int d = 0; d < BLK; ++d) acc[d] = 0.0f;
            for (int64_t c0 = 0; c0 < total; c0 += CHK) {
                const int n = (int) imin(CHK, total - c0);
                float cm = -INFINITY;
                for (int i = 0; i < n; ++i) {
                    const int64_t idx = c0 + i;
                    int64_t j = idx;
                    if (sel) {
                        const int32_t b = sel[(t * G + gi) * K + idx / BLK];
                        j = b < 0 ? -1 : (int64_t) b * BLK + idx % BLK;
                    }
                    float sv = -INFINITY;
                    if (j >= 0 && j <= pos) {
                        const uint16_t* kr = kc + (j * G + gi) * BLK;
                        float a = 0.0f;
                        for (int d = 0; d < BLK; ++d) a += qr[d] * orc_h2f(kr[d]);
                        sv = a * scale;
                    } else {
                        j = -1;
                    }
                    sc[i] = sv;
                    jj[i] = j;
                    cm = fmaxf(cm, sv);
                }
                const float nm = fmaxf(m, cm), corr = m == -INFINITY ? 0.0f : expf(m - nm);
                /* the device sums each of 128 lanes' weights i, i + 128, ... and then reduces; any order is float32
                 * reassociation */
                float ls = 0.0f;
                if (nm > -INFINITY)
                    for (int i = 0; i < n; ++i) {
                        sc[i] = sc[i] == -INFINITY ? 0.0f : expf(sc[i] - nm);
                        ls += sc[i];
                    }
                l = l * corr + ls;
                for (int d = 0; d < BLK; ++d) acc[d] *= corr;
                if (nm > -INFINITY)
                    for (int i = 0; i < n; ++i) {
                        if (jj[i] < 0) continue;
                        const uint16_t* vr = vc + (jj[i] * G + gi) * BLK;
                        for (int d = 0; d < BLK; ++d) acc[d] += sc[i] * orc_h2f(vr[d]);
                    }
                m = nm;
            }
            for (int d = 0; d < BLK; ++d) out[(t * H + hq) * BLK + d] = l > 0.0f ? acc[d] / l : 0.0f;
        }
    return 0;
}
ORC_API int orc_mm3_attend(const float* q, const uint16_t* kc, const uint16_t* vc, float* out, int64_t T, int64_t H, int64_t G, int64_t pos0,
                           float scale) {
    return orc_mm3_attend_sel(q, kc, vc, NULL, 0, out, T, H, G, pos0, scale);
}

/* MiniMax-M3's block indexer - kernels/llm/minimaxm3/mm3.cpp:59-116. Scores: bs [T][G][nblk] = the largest iq . ik_j over a
 * block's keys j <= pos (ik half [pos][128]); -inf for a block wholly past the row; + 1e30 for the `local` most recent
 * blocks (b + local > pos / 128), which therefore always win. */
ORC_API void orc_mm3_idx_scores(const float* iq, const uint16_t* ik, float* bs, int64_t T, int64_t G, int64_t nblk, int64_t pos0, int64_t local) {
    enum { BLK = 128 };
    for (int64_t t = 0; t < T; ++t)
        for (int64_t gi = 0; gi < G; ++gi)
            for (int64_t b = 0; b < nblk; ++b) {
                const int64_t pos = pos0 + t;
                const float* qv = iq + (t * G + gi) * BLK;
                float m = -INFINITY;
                for (int64_t j = b * BLK; j < (b + 1) * BLK && j <= pos; ++j) {
                    float sv = 0.0f;
                    for (int d = 0; d < BLK; ++d) sv += qv[d] * orc_h2f(ik[j * BLK + d]);
                    m = fmaxf(m, sv);
                }
                if (b * BLK > pos) m = -INFINITY;
                else if (b + local > pos / BLK) m = m + 1e30f;
                bs[(t * G + gi) * nblk + b] = m;
            }
}
/* Top K blocks a row, best first, the lowest index of equal scores; -1 once nothing finite is left. The scores picked
 * are overwritten with -inf, as the device does (:91-116). */
ORC_API void orc_mm3_idx_topk(float* bs, int32_t* sel, int64_t T, int64_t G, int64_t nblk, int64_t K) {
    for (int64_t row = 0; row < T * G; ++row) {
        float* sc = bs + row * nblk;
        for (int64_t k = 0; k < K; ++k) {
            float best = -INFINITY;
            for (int64_t b = 0; b < nblk; ++b) best = fmaxf(best, sc[b]);
            int32_t at = -1;
            if (best > -INFINITY)
                for (int64_t b = 0; b < nblk; ++b)
                    if (sc[b] == best) { at = (int32_t) b; break; }
            sel[row * K + k] = at;
            if (at >= 0) sc[at] = -INFINITY;
        }
    }
}

/* ------------------------------------------------------------------------------------------------ MLA */

/* ggml's rope_yarn angle for pair i0 of n_dims at position p, the angle by repeated products -
 * kernels/llm/deepseek2/ds2.cpp:15-34 */
static float yarn_ramp(float low, float high, int i0) {
    const float y = ((float) (i0 / 2) - low) / fmaxf(0.001f, high - low);
    return 1.0f - fminf(1.0f, fmaxf(0.0f, y));
}
static void yarn_cs(float p, int i0, int n_dims, float freq_base, float freq_scale, float ext_factor, float mscale, float corr0, float corr1,
                    float* c, float* s) {
    const float theta_scale = powf(freq_base, -2.0f / (float) n_dims);
    float theta_extrap = p;
    for (int k = 0; k < i0 / 2; ++k) theta_extrap *= theta_scale;
    const float theta_interp = freq_scale * theta_extrap;
    float theta = theta_interp;
    if (ext_factor != 0.0f) {
        const float ramp_mix = yarn_ramp(corr0, corr1, i0) * ext_factor;
        theta = theta_interp * (1 - ramp_mix) + theta_extrap * ramp_mix;
    }
    *c = cosf(theta) * mscale;
    *s = sinf(theta) * mscale;
}

/* the latent cache's rows pos0.. : [RMSnorm(kv[:L]) w | YaRN-rope(kv[L:L+R])] as half -
 * kernels/llm/deepseek2/ds2.cpp:85-112. The device sums the squares in a work-group reduction of unspecified order;
 * here they are summed in float64 and rounded once (any float32 order is within reassociation error of it, so a
 * stored half may differ from a device's in its last bit) */
ORC_API int orc_ds2_kv_store(const float* kv, const float* w, float eps, uint16_t* cache, int64_t T, int64_t L, int64_t R, int64_t pos0,
                             float freq_base, float freq_scale, float ext_factor, float mscale, float corr0, float corr1) {
    if (R % 2) return -1;
    for (int64_t t = 0; t < T; ++t) {
        const float* xr = kv + t * (L + R);
        double ssd = 0.0;
        for (int64_t i = 0; i < L; ++i) ssd += (double) xr[i] * (double) xr[i];
        const float ss = (float) ssd;
        const float inv = 1.0f / sqrtf(ss / (float) L + eps);
        uint16_t* o = cache + (pos0 + t) * (L + R);
        for (int64_t i = 0; i < L; ++i) o[i] = orc_f2h(xr[i] * inv * w[i]);
        for (int64_t i = 0; i < R / 2; ++i) {
            const int i0 = (int) (2 * i);
            float c, s;
            yarn_cs((float) (pos0 + t), i0, (int) R, freq_base, freq_scale, ext_factor, mscale, corr0, corr1, &c, &s);
            const float x0 = xr[L + i0], x1 = xr[L + i0 + 1];
            o[L + i0] = orc_f2h(x0 * c - x1 * s);
            o[L + i0 + 1] = orc_f2h(x0 * s + x1 * c);
        }
    }
    return 0;
}

/* ggml's YaRN rope in place on the rotated part of every head, a copy of that part to out where given -
 * kernels/llm/deepseek2/ds2.cpp:59-83 */
ORC_API int orc_ds2_rope(float* x, int64_t T, int64_t H, int64_t row, int64_t head, int64_t off, int64_t n_dims, int64_t pos0, float freq_base,
                         float freq_scale, float ext_factor, float mscale, float corr0, float corr1, float* out, int64_t out_row, int64_t out_head) {
    if (n_dims % 2) return -1;
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < H; ++h)
            for (int64_t i = 0; i < n_dims / 2; ++i) {
                const int i0 = (int) (2 * i);
                float c, s;
                yarn_cs((float) (pos0 + t), i0, (int) n_dims, freq_base, freq_scale, ext_factor, mscale, corr0, corr1, &c, &s);
                float* v = x + t * row + h * head + off + i0;
                const float x0 = v[0], x1 = v[1];
                const float y0 = x0 * c - x1 * s, y1 = x0 * s + x1 * c;
                v[0] = y0;
                v[1] = y1;
                if (out) {
                    float* o = out + t * out_row + h * out_head + i0;
                    o[0] = y0;
                    o[1] = y1;
                }
            }
    return 0;
}

/* GLM's DSA indexer - kernels/llm/glm5next/glm.cpp:876-1019 */
ORC_API void orc_idx_pool(float* ring, const float* ik, const float* ig, const float* ape, float* pooled, int64_t pos0, int64_t T, int64_t D) {
    const int64_t j_lo = pos0 / 4, j_hi = (pos0 + T) / 4;
    for (int64_t j = j_lo; j < j_hi; ++j)
        for (int64_t c = 0; c < D; ++c) {
            float lg[4], kv[4], mx = -INFINITY;
            for (int m = 0; m < 4; ++m) {
                const int64_t p = 4 * j + m;
                const float* k = p >= pos0 ? ik + (p - pos0) * D : ring + (p % 8) * 2 * D;
                const float* gg = p >= pos0 ? ig + (p - pos0) * D : ring + (p % 8) * 2 * D + D;
                kv[m] = k[c];
                lg[m] = gg[c] + ape[m * D + c];
                mx = fmaxf(mx, lg[m]);
            }
            float s = 0.f, acc = 0.f;
            for (int m = 0; m < 4; ++m) {
                const float e = expf(lg[m] - mx);
                s += e;
                acc += e * kv[m];
            }
            pooled[j * D + c] = acc / s;
        }
    const int64_t first = pos0 > pos0 + T - 8 ? pos0 : pos0 + T - 8;
    for (int64_t p = first; p < pos0 + T; ++p)
        for (int64_t c = 0; c < D; ++c) {
            ring[(p % 8) * 2 * D + c] = ik[(p - pos0) * D + c];
            ring[(p % 8) * 2 * D + D + c] = ig[(p - pos0) * D + c];
        }
}

ORC_API void orc_idx_score(const float* S, const float* w, float* score, int64_t T, int64_t H, int64_t j0, int64_t n, int64_t ld, int64_t pos0) {
    for (int64_t r = 0; r < T; ++r)
        for (int64_t jj = 0; jj < n; ++jj) {
            const int64_t j = j0 + jj, nv = (pos0 + r + 1) / 4;
            float s = -INFINITY;
            if (j < nv) {
                s = 0.f;
                for (int64_t h = 0; h < H; ++h) s += fmaxf(S[(r * H + h) * n + jj], 0.f) * w[r * H + h];
            }
            score[r * ld + j] = s;
        }
}

/* the K highest of a row as positions in ascending order, ties at the K-th value to the lowest positions (the radix
 * select of glm.cpp:940-1019 restated as what it selects: count the keys above the K-th, take those and the first
 * remaining equal ones) */
ORC_API void orc_topk(const float* score, int32_t* sel, int64_t T, int64_t n, int64_t ld, int64_t K) {
    for (int64_t r = 0; r < T; ++r) {
        const float* row = score + r * ld;
        uint32_t* key = (uint32_t*) malloc((size_t) (n > 0 ? n : 1) * sizeof(uint32_t));
        for (int64_t j = 0; j < n; ++j) {
            uint32_t u;
            memcpy(&u, row + j, 4);
            key[j] = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
        }
        /* the K-th largest key, digit by digit from the top */
        uint32_t prefix = 0, mask = 0, need = (uint32_t) K;
        for (int shift = 24; shift >= 0; shift -= 8) {
            uint32_t hist[256] = {0};
            for (int64_t j = 0; j < n; ++j)
                if ((key[j] & mask) == prefix) hist[(key[j] >> shift) & 255]++;
            uint32_t above = 0;
            int d = 255;
            for (; d > 0; --d) {
                if (above + hist[d] >= need) break;
                above += hist[d];
            }
            prefix |= (uint32_t) d << shift;
            mask |= 255u << shift;
            need -= above;
        }
        int64_t at = 0;
        uint32_t ties = need;
        for (int64_t j = 0; j < n && at < K; ++j)
            if (key[j] > prefix || (key[j] == prefix && ties > 0)) {
                if (key[j] == prefix) --ties;
                sel[r * K + at++] = (int32_t) j;
            }
        free(key);
    }
}

/* q~ = k_b q_nope per (row, head): qa [T][H][L + R] = [q~ (L) | q_pe (R)] from q [T][H][nope + R], kb half [H][L][nope] -
 * kernels/llm/deepseek2/ds2.cpp:176-184 (a lane sums 8 products, 16 lanes reduced) */
ORC_API void orc_mla_absorb(const float* q, const uint16_t* kb, float* qa, int64_t T, int64_t H, int64_t L, int64_t R, int64_t NOPE) {
#pragma omp parallel for collapse(2)
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < H; ++h) {
            const float* qr = q + (t * H + h) * (NOPE + R);
            float* o = qa + (t * H + h) * (L + R);
            for (int64_t r = 0; r < L; ++r) {
                const uint16_t* w = kb + (h * L + r) * NOPE;
                float lane[16];
                for (int ln = 0; ln < 16; ++ln) {
                    float a = 0.0f;
                    for (int64_t f = 0; f < NOPE / 16; ++f) a += orc_h2f(w[ln * (NOPE / 16) + f]) * qr[ln * (NOPE / 16) + f];
                    lane[ln] = a;
                }
                for (int o2 = 8; o2 > 0; o2 >>= 1)
                    for (int ln = 0; ln < o2; ++ln) lane[ln] += lane[ln + o2];
                o[r] = lane[0];
            }
            for (int64_t f = 0; f < R; ++f) o[L + f] = qr[NOPE + f];
        }
}

/* The absorbed decode over the latent cache [n][L + R] half, per (row t, head h), the reference's order kept: 16
 * streams (stream s: cells s, s + 16, ...) each an online softmax with exp; merged with exp(m - mx); u = acc / sum -
 * kernels/llm/deepseek2/ds2.cpp:186-235. qa [T][H][L + R] (absorbed, float32); u [T][H][L]. A cell's score: each of 16
 * lanes sums its L/16 latent products then its R/16 rope products, the lanes added as a butterfly, x scale. */
ORC_API void orc_mla_decode_u(const float* qa, const uint16_t* cache, float* u, int64_t T, int64_t H, int64_t L, int64_t R, int64_t pos0,
                              float scale) {
    enum { NSG = 16, LANES = 16 };
    const int64_t CR = L + R, DL = L / LANES, DR = R / LANES;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < H; ++h) {
            const float* qv = qa + (t * H + h) * CR;
            const int64_t n = pos0 + t + 1;
            float* acc = (float*) calloc((size_t) (NSG * L), sizeof(float));
            float m[NSG], sum[NSG];
            for (int s = 0; s < NSG; ++s) {
                m[s] = -INFINITY;
                sum[s] = 0.0f;
                for (int64_t i = s; i < n; i += NSG) {
                    const uint16_t* row = cache + i * CR;
                    float lane[LANES];
                    for (int ln = 0; ln < LANES; ++ln) {
                        float d = 0.0f;
                        for (int64_t f = 0; f < DL; ++f) d += qv[ln * DL + f] * orc_h2f(row[ln * DL + f]);
                        for (int64_t f = 0; f < DR; ++f) d += qv[L + ln * DR + f] * orc_h2f(row[L + ln * DR + f]);
                        lane[ln] = d;
                    }
                    for (int o = LANES / 2; o > 0; o >>= 1)
                        for (int ln = 0; ln < o; ++ln) lane[ln] += lane[ln + o];
                    const float d = lane[0] * scale;
                    const float mn = fmaxf(m[s], d);
                    const float a = expf(m[s] - mn), b = expf(d - mn);
                    sum[s] = sum[s] * a + b;
                    for (int64_t f = 0; f < L; ++f) acc[s * L + f] = acc[s * L + f] * a + b * orc_h2f(row[f]);
                    m[s] = mn;
                }
            }
            float mx = -INFINITY, tot = 0.0f;
            for (int s = 0; s < NSG; ++s) mx = fmaxf(mx, m[s]);
            for (int s = 0; s < NSG; ++s) tot += m[s] == -INFINITY ? 0.0f : sum[s] * expf(m[s] - mx);
            float* o = u + (t * H + h) * L;
            for (int64_t f = 0; f < L; ++f) {
                float v = 0.0f;
                for (int s = 0; s < NSG; ++s) v += acc[s * L + f] * (m[s] == -INFINITY ? 0.0f : expf(m[s] - mx));
                o[f] = v / tot;
            }
            free(acc);
        }
}

/* Q6_K (210 bytes a 256 values): ql [128], qh [64], int8 scales [16], half d. The 32 values of block half n, quarter gq at
 * l = 0..31: (low or high nibble of ql[64 n + (gq & 1) 32 + l]) | two bits of qh[32 n + l] << 4, less 32, times d x
 * scale[8 n + 2 gq + l / 16], the products in that order - kernels/llm/deepseek2/ds2.cpp:117-134. Columns [32 k, 32 k + 32)
 * of a 512-wide row (two blocks). */
static void q6k_cols32(const uint8_t* row, int k, float* v) {
    const uint8_t* b = row + (k / 8) * 210;
    const int j = (k % 8) * 32, n = j / 128, gq = (j % 128) / 32;
    uint16_t dh;
    memcpy(&dh, b + 208, 2);
    const float d = orc_h2f(dh);
    const uint8_t* ql = b + 64 * n + (gq & 1) * 32;
    const uint8_t* qh = b + 128 + 32 * n;
    const int shift = 2 * gq;
    for (int l = 0; l < 32; ++l) {
        const int lo = gq < 2 ? (ql[l] & 0xF) : (ql[l] >> 4);
        const int q = (lo | (((qh[l] >> shift) & 3) << 4)) - 32;
        v[l] = d * (float) (int8_t) b[192 + 8 * n + 2 * gq + l / 16] * (float) q;
    }
}

/* a Q6_K row of 512 widened to float32 (the rule above) */
ORC_API void orc_q6k_row512(const uint8_t* row, float* out) {
    for (int k = 0; k < 16; ++k) q6k_cols32(row, k, out + 32 * k);
}

/* q~ over kv_b as the file stores it (Q6_K, per head 128 k rows then 128 v rows, each [512]): q~[c] = sum_i q_nope[i]
 * k_i[c], 16 streams (stream s: rows s, s + 16, ..) added in stream order - kernels/llm/deepseek2/ds2.cpp:157-173 */
ORC_API void orc_mla_absorb_q6k(const float* q, const uint8_t* kvb, float* qa, int64_t T, int64_t H) {
    enum { L = 512, R = 64, NOPE = 128, V = 128, NSG = 16 };
#pragma omp parallel for collapse(2)
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < H; ++h) {
            const float* qr = q + (t * H + h) * (NOPE + R);
            float* o = qa + (t * H + h) * (L + R);
            float part[NSG][L];
            memset(part, 0, sizeof(part));
            for (int s = 0; s < NSG; ++s)
                for (int i = s; i < NOPE; i += NSG) {
                    float row[L];
                    orc_q6k_row512(kvb + ((size_t) h * (NOPE + V) + i) * 420, row);
                    for (int c = 0; c < L; ++c) part[s][c] += qr[i] * row[c];
                }
            for (int c = 0; c < L; ++c) {
                float a = 0.0f;
                for (int s = 0; s < NSG; ++s) a += part[s][c];
                o[c] = a;
            }
            for (int f = 0; f < R; ++f) o[L + f] = qr[NOPE + f];
        }
}

/* out = v_b u over the Q6_K v rows: a lane 32 columns in order, 16 lanes reduced - kernels/llm/deepseek2/ds2.cpp:237-246 */
ORC_API void orc_mla_vb_q6k(const float* u, const uint8_t* kvb, float* out, int64_t T, int64_t H) {
    enum { L = 512, NOPE = 128, V = 128 };
#pragma omp parallel for collapse(2)
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < H; ++h)
            for (int64_t r = 0; r < V; ++r) {
                float row[L], lane[16];
                orc_q6k_row512(kvb + ((size_t) h * (NOPE + V) + NOPE + r) * 420, row);
                const float* uu = u + (t * H + h) * L;
                for (int ln = 0; ln < 16; ++ln) {
                    float a = 0.0f;
                    for (int f = 0; f < 32; ++f) a += row[ln * 32 + f] * uu[ln * 32 + f];
                    lane[ln] = a;
                }
                for (int o = 8; o > 0; o >>= 1)
                    for (int ln = 0; ln < o; ++ln) lane[ln] += lane[ln + o];
                out[(t * H + h) * V + r] = lane[0];
            }
}

/* out [T][H][V] = v_b u: vb half [H][V][L] - kernels/llm/deepseek2/ds2.cpp:237-255 (lane ln sums columns
 * (k*16 + ln)*8 .. +8 for k = 0..3, then the 16 lanes are reduced) */
ORC_API void orc_mla_vb(const float* u, const uint16_t* vb, float* out, int64_t T, int64_t H, int64_t L, int64_t V) {
#pragma omp parallel for collapse(2)
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < H; ++h)
            for (int64_t r = 0; r < V; ++r) {
                const uint16_t* vr = vb + (h * V + r) * L;
                const float* uu = u + (t * H + h) * L;
                float lane[16];
                for (int ln = 0; ln < 16; ++ln) {
                    float a = 0.0f;
                    for (int64_t k = 0; k < L / 128; ++k)
                        for (int f = 0; f < 8; ++f) a += orc_h2f(vr[(k * 16 + ln) * 8 + f]) * uu[(k * 16 + ln) * 8 + f];
                    lane[ln] = a;
                }
                for (int o = 8; o > 0; o >>= 1)
                    for (int ln = 0; ln < o; ++ln) lane[ln] += lane[ln + o];
                out[(t * H + h) * V + r] = lane[0];
            }
}

/* float64 closed form of the absorbed decode: u[t][h][:] = softmax_i(scale qa . c_i) c_i[:L] over cells 0..pos0 + t.
 * cache rows `cr` halfs apart hold [L (+ R)]; qa rows hold QW = L + R values (R may be 0: GLM's latent-only MLA) */
ORC_API void orc_mla_f64(const float* qa, const uint16_t* cache, double* u, int64_t T, int64_t H, int64_t L, int64_t R, int64_t pos0,
                         double scale) {
    const int64_t CR = L + R;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < H; ++h) {
            const float* qv = qa + (t * H + h) * CR;
            const int64_t n = pos0 + t + 1;
            double* s = (double*) malloc(sizeof(double) * (size_t) n);
            double mx = -INFINITY;
            for (int64_t i = 0; i < n; ++i) {
                const uint16_t* row = cache + i * CR;
                double a = 0.0;
                for (int64_t f = 0; f < CR; ++f) a += (double) qv[f] * (double) orc_h2f(row[f]);
                s[i] = a * scale;
                if (s[i] > mx) mx = s[i];
            }
            double* o = u + (t * H + h) * L;
            for (int64_t f = 0; f < L; ++f) o[f] = 0.0;
            double l = 0.0;
            for (int64_t i = 0; i < n; ++i) {
                const double e = exp(s[i] - mx);
                l += e;
                const uint16_t* row = cache + i * CR;
                for (int64_t f = 0; f < L; ++f) o[f] += e * (double) orc_h2f(row[f]);
            }
            for (int64_t f = 0; f < L; ++f) o[f] /= l;
            free(s);
        }
}

/* GLM-5.3's latent-only MLA, two passes: every score (qa . c_i) scale, their maximum, then w_i = exp(d_i - mx),
 * u = sum w_i c_i / sum w_i - kernels/llm/glm5next/glm.cpp:1129-1183. q8 != 0: rows [L/32 half scales][L int8], value
 * h2f(d_b) q. */
ORC_API void orc_glm_mla_attend_sel(const float* qa, const uint8_t* cache, int q8, float* u, int64_t T, int64_t H, int64_t L, int64_t pos0,
                                    float scale, const int32_t* sel, const int32_t* sel_cnt, int64_t K) {
    const int64_t nb = L / 32, rb = q8 ? nb * 2 + L : 2 * L;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < H; ++h) {
            const float* qv = qa + (t * H + h) * L;
            /* a row's cells: every earlier one (sel_cnt NULL or negative), or the pools sel[t][0, sel_cnt[t]) of 4 cells
             * each and the row's incomplete pool 4 ((p + 1) / 4) .. p - kernels/llm/glm5next/glm.cpp:1062-1067,1095-1102 */
            const int64_t p = pos0 + t, ns = sel_cnt ? sel_cnt[t] : -1, tail0 = 4 * ((p + 1) / 4);
            const int64_t n = ns < 0 ? p + 1 : 4 * ns + (p + 1 - tail0);
#define ORC_CELL(i) (ns < 0 ? (i) : (i) < 4 * ns ? 4 * (int64_t) sel[t * K + (i) / 4] + (i) % 4 : tail0 + ((i) - 4 * ns))
            float* s = (float*) malloc(sizeof(float) * (size_t) (n > 0 ? n : 1));
            float* c = (float*) malloc(sizeof(float) * (size_t) L);
            float mx = -INFINITY;
            for (int64_t i = 0; i < n; ++i) {
                const uint8_t* row = cache + ORC_CELL(i) * rb;
                float a = 0.0f;
                for (int64_t f = 0; f < L; ++f) {
                    const float cv = q8 ? orc_h2f(ld16(row + 2 * (f / 32))) * (float) (int8_t) row[nb * 2 + f] : orc_h2f(ld16(row + 2 * f));
                    a += qv[f] * cv;
                }
                s[i] = a * scale;
                mx = fmaxf(mx, s[i]);
            }
            float* o = u + (t * H + h) * L;
            for (int64_t f = 0; f < L; ++f) o[f] = 0.0f;
            float tot = 0.0f;
            for (int64_t i = 0; i < n; ++i) {
                const uint8_t* row = cache + ORC_CELL(i) * rb;
                const float w = expf(s[i] - mx);
                tot += w;
                for (int64_t f = 0; f < L; ++f) {
                    c[f] = q8 ? orc_h2f(ld16(row + 2 * (f / 32))) * (float) (int8_t) row[nb * 2 + f] : orc_h2f(ld16(row + 2 * f));
                    o[f] += w * c[f];
                }
            }
#undef ORC_CELL
            for (int64_t f = 0; f < L; ++f) o[f] = tot > 0.0f ? o[f] / tot : 0.0f;
            free(s);
            free(c);
        }
}
ORC_API void orc_glm_mla_attend(const float* qa, const uint8_t* cache, int q8, float* u, int64_t T, int64_t H, int64_t L, int64_t pos0,
                                float scale) {
    orc_glm_mla_attend_sel(qa, cache, q8, u, T, H, L, pos0, scale, NULL, NULL, 0);
}

/* GLM-5.3's dense MLA over a float32 latent cache c [n][L], two passes (the largest score, then the weights and the sum)
 * - kernels/llm/glm5next/glm.cpp:782-812. The reference sums a score's L products across 256 work-items (an order SYCL
 * leaves open); here feature-ascending in float32. */
ORC_API void orc_glm_mla_attend_f32(const float* qa, const float* c, float* u, int64_t T, int64_t H, int64_t L, int64_t pos0, float scale) {
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < H; ++h) {
            const float* qr = qa + (t * H + h) * L;
            const int64_t n = pos0 + t + 1;
            float mx = -INFINITY;
            for (int64_t s = 0; s < n; ++s) {
                float dot = 0.0f;
                for (int64_t r = 0; r < L; ++r) dot += qr[r] * c[s * L + r];
                mx = fmaxf(mx, dot * scale);
            }
            float* o = u + (t * H + h) * L;
            for (int64_t r = 0; r < L; ++r) o[r] = 0.0f;
            float sum = 0.0f;
            for (int64_t s = 0; s < n; ++s) {
                float dot = 0.0f;
                for (int64_t r = 0; r < L; ++r) dot += qr[r] * c[s * L + r];
                const float p = expf(dot * scale - mx);
                sum += p;
                for (int64_t r = 0; r < L; ++r) o[r] += p * c[s * L + r];
            }
            for (int64_t r = 0; r < L; ++r) o[r] /= sum;
        }
}

/* out [n][L] half = the q8 latent rows idx[i] of src widened: half(h2f(scale) x (float) q) - kernels/llm/glm5next/glm.cpp:1301-1325 */
ORC_API void orc_glm_gather_q8_h(const uint8_t* src, const int32_t* idx, uint16_t* out, int64_t n, int64_t L) {
    const int64_t nb = L / 32, rb = nb * 2 + L;
    for (int64_t i = 0; i < n; ++i) {
        const uint8_t* row = src + (int64_t) idx[i] * rb;
        for (int64_t f = 0; f < L; ++f) out[i * L + f] = orc_f2h(orc_h2f(ld16(row + 2 * (f / 32))) * (float) (int8_t) row[nb * 2 + f]);
    }
}

/* Each row's cells as a list: idx [T][NC], n [T] - kernels/llm/glm5next/glm.cpp:1023-1039. sel_cnt NULL or sel_cnt[t] < 0:
 * the cells 0 .. p; else the 4 tokens of each listed pool, then the incomplete pool's tokens 4 ((p + 1) / 4) .. p. */
ORC_API void orc_glm_mla_cells(const int32_t* sel, const int32_t* sel_cnt, int64_t T, int64_t K, int64_t pos0, int32_t* idx, int32_t* n, int64_t NC) {
    for (int64_t t = 0; t < T; ++t) {
        const int64_t p = pos0 + t, ns = sel_cnt ? sel_cnt[t] : -1, tail0 = 4 * ((p + 1) / 4);
        const int64_t cnt = ns < 0 ? p + 1 : 4 * ns + (p + 1 - tail0);
        for (int64_t i = 0; i < NC; ++i) {
            int64_t c = 0;
            if (i < cnt) c = ns < 0 ? i : i < 4 * ns ? 4 * (int64_t) sel[t * K + i / 4] + i % 4 : tail0 + (i - 4 * ns);
            idx[t * NC + i] = (int32_t) c;
        }
        n[t] = (int32_t) (cnt < NC ? cnt : NC);
    }
}

/* Row softmax of S [R H][NC] in place over the first n[r] cells of row r's heads, scaled; 0 behind them -
 * kernels/llm/glm5next/glm.cpp:1041-1060 (float32 throughout; the reference adds a work-group's terms in tree order,
 * here in index order) */
ORC_API void orc_glm_softmax_masked(float* S, int64_t R, int64_t H, int64_t NC, const int32_t* n, float scale) {
    for (int64_t rh = 0; rh < R * H; ++rh) {
        float* row = S + rh * NC;
        const int64_t m = n[rh / H];
        float mx = -INFINITY, sum = 0.0f;
        for (int64_t i = 0; i < m; ++i) mx = fmaxf(mx, row[i] * scale);
        for (int64_t i = 0; i < m; ++i) sum += expf(row[i] * scale - mx);
        for (int64_t i = 0; i < NC; ++i) row[i] = i < m ? expf(row[i] * scale - mx) / sum : 0.0f;
    }
}

/* ------------------------------------------------------------------------------------ norm + rotary positions */

/* kernels/llm/qwen35/q35.cpp:220-254 (w != NULL: RMS norm first), :256-279 (w == NULL: ns_q35_rope), :350-386 (pos3 != NULL:
 * each row at its own (t, h, w) positions, interleaved sections s0, s1, s2). Rotate-half over the first n_rot features:
 * pair (i, i + n_rot / 2), angle pos * theta^(-2 k / n_rot), every product in float32. The reference sums the squares as 16
 * lane sums (i = l, l + 16, ...) added by a group reduction; here the lane sums are added in lane order. */
ORC_API int orc_q35_norm_rope(const float* src, int64_t ss, int64_t hs, float* dst, int64_t ds, int64_t T, int64_t H, int64_t D, const float* w,
                              float eps, int64_t n_rot, float theta, int64_t p0, const int32_t* pos3, int64_t s0, int64_t s1, int64_t s2) {
    if (D % 16 != 0 || n_rot > D || n_rot % 2 || (pos3 && s0 + s1 + s2 <= 0)) return -1;
    const int64_t hr = n_rot / 2, sect = s0 + s1 + s2;
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < H; ++h) {
            const float* x = src + t * ss + h * hs;
            float* y = dst + t * ds + h * D;
            float inv = 1.0f;
            if (w) {
                float lane[16], s = 0.0f;
                for (int l = 0; l < 16; ++l) {
                    lane[l] = 0.0f;
                    for (int64_t i = l; i < D; i += 16) lane[l] += x[i] * x[i];
                }
                for (int l = 0; l < 16; ++l) s += lane[l];
                inv = 1.0f / sqrtf(s / (float) D + eps);
            }
            for (int64_t i = 0; i < D; ++i) {
                const float v = w ? x[i] * inv * w[i] : x[i];
                if (i < n_rot) {
                    const int64_t k = i < hr ? i : i - hr;
                    float pos = (float) (p0 + t);
                    if (pos3) {
                        const int64_t sec = k % sect;
                        const int c = (sec % 3 == 1 && sec < 3 * s1) ? 1 : (sec % 3 == 2 && sec < 3 * s2) ? 2 : 0;
                        pos = (float) pos3[t * 3 + c];
                    }
                    const float a = pos * powf(theta, -2.0f * (float) k / (float) n_rot);
                    const float c = cosf(a), sn = sinf(a);
                    const int64_t o = i < hr ? i + hr : i - hr;
                    const float other = w ? x[o] * inv * w[o] : x[o];
                    y[i] = i < hr ? v * c - other * sn : v * c + other * sn;
                } else {
                    y[i] = v;
                }
            }
        }
    return 0;
}

/* kernels/llm/museglimmer/mg.cpp:157-190: RMS norm, then rope 0 none, 1 adjacent pairs (2i, 2i + 1), 2 halves (i, i + D / 2)
 * over all D, angle pos * theta^(-2 i / D). y may be x (a pair is read before it is written). */
ORC_API int orc_mg_norm_rope(const float* x, int64_t xs, float* y, int64_t ys, int64_t T, int64_t H, int64_t D, const float* w, float eps, int rope,
                             float theta, int64_t p0) {
    if (D % 32 != 0) return -1;
    for (int64_t t = 0; t < T; ++t)
        for (int64_t h = 0; h < H; ++h) {
            const float* xr = x + t * xs + h * D;
            float* yr = y + t * ys + h * D;
            float lane[16], s = 0.0f;
            for (int l = 0; l < 16; ++l) {
                lane[l] = 0.0f;
                for (int64_t i = l; i < D; i += 16) lane[l] += xr[i] * xr[i];
            }
            for (int l = 0; l < 16; ++l) s += lane[l];
            const float inv = 1.0f / sqrtf(s / (float) D + eps);
            const float pos = (float) (p0 + t);
            for (int64_t i = 0; i < D / 2; ++i) {
                const int64_t i0 = rope == 2 ? i : 2 * i, i1 = rope == 2 ? i + D / 2 : 2 * i + 1;
                const float a0 = xr[i0] * inv * w[i0], a1 = xr[i1] * inv * w[i1];
                if (rope) {
                    const float a = pos * powf(theta, -2.0f * (float) i / (float) D);
                    const float c = cosf(a), sn = sinf(a);
                    yr[i0] = a0 * c - a1 * sn;
                    yr[i1] = a0 * sn + a1 * c;
                } else {
                    yr[i0] = a0;
                    yr[i1] = a1;
                }
            }
        }
    return 0;
}

/* kernels/llm/minimaxm3/mm3.cpp:18-35 (w == NULL: in-place rotate-half, the angle of pair i = pos multiplied i times by
 * base^(-2 / n_rot)) and silo/moe.cpp:477-497 (w != NULL: RMS norm as 1 / sqrt first; half != NULL: the result also stored
 * as half; rot == 0 with w == NULL: a plain half store, the token's v rows). One head row of HD floats. */
ORC_API int orc_mm3_norm_rope_row(float* p, const float* w, uint16_t* half, int rot, int64_t HD, int64_t n_rot, int64_t pos, float base, float eps) {
    if (n_rot % 2 || n_rot > HD) return -1;
    const int64_t hr = n_rot / 2;
    const float ts = n_rot > 0 ? powf(base, -2.0f / (float) n_rot) : 1.0f;
    float inv = 1.0f;
    if (w) {
        float sq = 0.0f;
        for (int64_t i = 0; i < HD; ++i) sq += p[i] * p[i];
        inv = 1.0f / sqrtf(sq / (float) HD + eps);
    }
    float* out = (float*) malloc((size_t) HD * sizeof(float));
    for (int64_t i = 0; i < HD; ++i) {
        const float me = w ? p[i] * inv * w[i] : p[i];
        if (rot && i < n_rot) {
            const int64_t k = i % hr, o = i < hr ? i + hr : i - hr;
            float th = (float) pos;
            for (int64_t j = 0; j < k; ++j) th *= ts;
            const float c = cosf(th), s = sinf(th);
            const float them = w ? p[o] * inv * w[o] : p[o];
            out[i] = i < hr ? me * c - them * s : them * s + me * c;
        } else {
            out[i] = me;
        }
    }
    for (int64_t i = 0; i < HD; ++i) {
        if (w || rot) p[i] = out[i];
        if (half) half[i] = orc_f2h(out[i]);
    }
    free(out);
    return 0;
}

/* ------------------------------------------------------------------------------------------------ comparisons */

/* max |a - b|, relative L2 sqrt(sum (a-b)^2 / sum b^2) and cosine, as the reference's `kernels` check reports them
 * (llm/deepseek2/src/tools.rs:25-36); a float32, b float64 */
ORC_API void orc_compare(const float* a, const double* b, int64_t n, double* max_abs, double* rel_l2, double* cosine) {
    double ab = 0, aa = 0, bb = 0, dd = 0, mx = 0;
    for (int64_t i = 0; i < n; ++i) {
        const double x = a[i], y = b[i], d = fabs(x - y);
        ab += x * y;
        aa += x * x;
        bb += y * y;
        dd += (x - y) * (x - y);
        if (d > mx || d != d) mx = d != d ? INFINITY : d;
    }
    *max_abs = mx;
    *rel_l2 = sqrt(dd / fmax(bb, 1e-30));
    *cosine = ab / fmax(sqrt(aa) * sqrt(bb), 1e-30);
}

ORC_API int orc_threads(void) {
    int n = 1;
#ifdef _OPENMP
#pragma omp parallel
    {
#pragma omp master
        n = omp_get_num_threads();
    }
#endif
    return n;
}
