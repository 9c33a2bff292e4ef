/* ns_attn.h - the LLM attention path of libnextsycl-llm.so on one AMD MI355X (gfx950): KV-cache stores, split-K decode
 * (one row, or the few rows of a speculative verify pass), causal flash-attention prefill. (MLA: ns_mla.h.)
 *
 * The entry points named ns_q35_*, ns_mg_*, ns_llm_minimaxm3_* are the ones the
 * reference engines bind by name (llm/<arch>/src/ffi.rs) - same names, argument order, layouts and error behaviour, so
 * an engine's ffi table resolves against this library unchanged. Each declaration cites the reference interface it
 * replaces. The ns_attn_* entry points are this library's own: the same operations with typed
 * (f32 / f16 / bf16) query and output rows, any G = Hq / Hkv, either cache layout and a bfloat16 cache form.
 *
 * Conventions (reference: kernels/llm/qwen35/q35.h:1-4): rows q/out are [T][Hq*D]; row t sits at absolute position
 * p0 + t and sees keys 0 .. p0 + t (causal); query head hq reads key head hq / (Hq / Hkv). Everything is queued on the
 * ns_gpu's compute stream and returns at once; 0, or -1 with the reason in ns_last_error(). The caller owns every
 * buffer; `scratch` may be NULL only when the matching *_scratch() returns 0. No call allocates device memory.
 *
 * Cache forms `kt` (reference: llm/qwen35/src/engine.rs:44-60, kernels/llm/qwen35/silo/attn.cpp:43-46):
 *   0  half       [D] half                                  2 D bytes a (head, position)
 *   1  q8_0       [D int8][D/32 half scales]                D + D/16 bytes   (D 128: 136, D 256: 272)
 *   2  q4_0       [D/2 bytes][D/32 half scales]             D/2 + D/16 bytes (D 128: 72,  D 256: 144)
 *   3  bfloat16   [D] bfloat16 (this library's addition)    2 D bytes
 * Cache layouts: head-major [Hkv][cap][row] (qwen35, museglimmer: slot = position, or position % cap for a ring) and
 * position-major [position][Hkv][row] (minimaxm3: kernels/llm/minimaxm3/mm3.h:33-36).
 */
#ifndef NS_ATTN_H
#define NS_ATTN_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ns_gpu ns_gpu;

/* element types of query / output rows for the typed entry points */
#define NS_F32 0
#define NS_F16 1
#define NS_BF16 2
/* cache forms */
#define NS_KV_F16 0
#define NS_KV_Q8_0 1
#define NS_KV_Q4_0 2
#define NS_KV_BF16 3

/* ---- KV-cache stores ------------------------------------------------------------------------------------------ */

/* float32 rows k [T, Hkv x D] (ks floats apart) and v (vs apart) into the half caches [Hkv][cap][D] at positions
 * p0.. ; -1 past the capacity. Replaces: kernels/llm/qwen35/q35.h:55-57 (q35.cpp:573-588) */
int ns_q35_kv_store(ns_gpu* g, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D, int64_t cap, int64_t p0,
                    void* kc, void* vc);
/* the same rows as q8_0 (kt 1) or q4_0 (kt 2) rows, bit for bit ggml's quantize_row_q8_0_ref / _q4_0_ref with the
 * scales behind the row's values; D a multiple of 32 (the reference: 256 only). Replaces:
 * kernels/llm/qwen35/q35.h:37-42 (q35.cpp:281-326) */
int ns_q35_kv_store_q(ns_gpu* g, int kt, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D, int64_t cap,
                      int64_t p0, void* kc, void* vc);
/* float32 rows k, v [T, Hkv x D] into half ring caches, slot (p0 + t) % cap. Replaces: kernels/llm/museglimmer/mg.h:25-26
 * (mg.cpp:192-206) */
int ns_mg_kv_store(ns_gpu* g, const float* k, const float* v, int64_t T, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, void* kc, void* vc);
/* this library's typed store: any cache form (kt 0..3), ring != 0 for slot = position % cap (forms 0 and 3 only) */
int ns_attn_kv_store(ns_gpu* g, int kt, int ring, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D,
                     int64_t cap, int64_t p0, void* kc, void* vc);
/* n cache rows of form kt (`stride` bytes apart) widened to float32 [n][D] exactly as the attention kernels read them
 * into float32 (kernels/llm/qwen35/q35.cpp:19-25): the check of the byte formats. This library's own */
int ns_attn_kv_dequant(ns_gpu* g, int kt, const void* rows, int64_t n, int64_t D, int64_t stride, float* out);
/* The rows of positions [from, to) of every head moved between two caches of `row_bytes`-byte rows, head-major
 * [heads][cap][row]: position p sits in slot (p - base) % cap of each. A ring is base 0, cap its slots; position
 * order (a checkpoint's buffer) is base `from`, cap to - from. to - from may not pass either capacity. One launch for
 * every head; queued like every call. Replaces the host loops of one or two copies a head in the engines' save /
 * restore / copy_session (llm/museglimmer/src/engine.rs:1334-1346,1475-1528, llm/qwen35/src/engine.rs:2977-3011):
 * the reference has no kernel for it */
int ns_attn_kv_rows_copy(ns_gpu* g, const void* src, int64_t scap, int64_t sbase, void* dst, int64_t dcap, int64_t dbase, int64_t heads,
                         int64_t row_bytes, int64_t from, int64_t to);
/* normalized 32-point Walsh-Hadamard transform of each block of 32 in place (a quantized cache's optional rotation).
 * Replaces: kernels/llm/qwen35/q35.h:43-45 (q35.cpp:328-348) */
int ns_q35_fwht32(ns_gpu* g, float* x, int64_t rows, int64_t n, int64_t stride);

/* ---- decode / verify attention (1..16 rows), split over the keys ------------------------------------------------ */

/* Typed decode: rows q [T][Hq*D] (element type qt, rows qs elements apart) at positions p0.. against caches of form kt;
 * pm 0 head-major [Hkv][cap][row] (slot = position % cap), 1 position-major [position][Hkv][row]; window win (<= 0:
 * all earlier keys); scale <= 0: 1/sqrt(D). out [T][Hq*D] of type qt. The keys are cut at absolute multiples of the
 * split size into ~512 work-groups, every row of the pass riding on each key tile (a key is read once for all T x G
 * rows of its key head); partials (values, max in log2 units, sum) [T][Hq][ns][D + 2] go through `scratch`
 * (ns_attn_decode_scratch floats, 8-byte aligned) and are merged by a second kernel. A row's result does not depend on
 * which other rows share its pass, bit for bit. D 128 or 256, T 1..16 */
int64_t ns_attn_decode_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0, int64_t win);
int ns_attn_decode_t(ns_gpu* g, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq,
                     int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, float scale, void* out, float* scratch);

/* ns_attn_decode_t without a scratch argument and without any allocation: the partials go through an array that is part
 * of the library's code object (NS_ATTN_STATIC_SCRATCH_FLOATS floats = 16 MiB, held by every GPU the library runs on
 * until the process ends; its address is looked up at ns_gpu_open). No counterpart in the reference: it is for callers
 * that cannot allocate - code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc. Same
 * arguments, same result bit for bit. -1 when ns_attn_decode_scratch(T, Hq, Hkv, D, p0, win) exceeds the array (take
 * ns_attn_decode_t with a buffer of the caller's then). Every call on a GPU shares that GPU's array: calls that overlap
 * on one GPU race */
#define NS_ATTN_STATIC_SCRATCH_FLOATS (4 << 20)
int ns_attn_decode_static(ns_gpu* g, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq,
                          int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, float scale, void* out);

/* Replaces: kernels/llm/qwen35/silo/silo.h:46-59 (silo/attn.cpp:375-435). The reference covers D 256 with 6 query
 * heads a key head and 1..8 rows; here D 128 or 256, any Hq a multiple of Hkv, 1..16 rows */
int ns_q35_attn_decode_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D);
int64_t ns_q35_attn_decode_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0);
int ns_q35_attn_decode(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D,
                       int64_t cap, int64_t p0, float* out, float* scratch);
int ns_q35_attn_decode_kv(ns_gpu* g, int kt, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv,
                          int64_t D, int64_t cap, int64_t p0, float* out, float* scratch);
/* Replaces: kernels/llm/museglimmer/silo/silo.h:50-56 (silo/attn.cpp:317-375): ring caches and a window */
int ns_mg_attn_decode_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D);
int64_t ns_mg_attn_decode_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0, int64_t win);
int ns_mg_attn_decode(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap,
                      int64_t p0, int64_t win, float* out, float* scratch);

/* ---- prompt (prefill) attention ---------------------------------------------------------------------------------- */

/* Typed causal flash attention of T rows at positions p0.. against caches that already hold positions 0 .. p0 + T - 1
 * (the engine stores a pass's keys first: llm/museglimmer/src/engine.rs:856-860). No scratch argument: a pass of few rows
 * over a long context is cut into key splits whose partials live in memory the library keeps per ns_gpu (calls on one
 * ns_gpu are ordered by its stream). D 128 or 256; kt 0 (half), 1 (q8_0), 2 (q4_0) or 3 (bfloat16). 16-bit caches
 * 16-byte aligned; quantized ones 16-byte aligned at D 256 (272- / 144-byte rows) and 8-byte aligned at D 128 (136 / 72) */
int ns_attn_prompt_t(ns_gpu* g, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq,
                     int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, float scale, void* out);
/* Replaces: kernels/llm/museglimmer/silo/silo.h:44-48 (silo/attn.cpp:378-392) */
int ns_mg_attn_prompt_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D);
int ns_mg_attn_prompt(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap,
                      int64_t p0, int64_t win, float* out);
/* Replaces: kernels/llm/qwen35/silo/silo.h:43-45,57-58 (silo/attn.cpp:375-400); _kv: kt 0, 1, 2 (the reference: at D 256) */
int ns_q35_attn_prompt_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D);
int ns_q35_attn_prompt(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D,
                       int64_t cap, int64_t p0, float* out);
int ns_q35_attn_prompt_kv(ns_gpu* g, int kt, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv,
                          int64_t D, int64_t cap, int64_t p0, float* out);

/* nemotron-h's silo names of the same two passes (the reference: D 128, 16 query heads a key head, decode rows 1..8).
 * Replaces: kernels/llm/nemotronh/silo/nhs.h:60-69 (silo/attn.cpp:337-369) */
int ns_nhs_attn_prompt_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D);
int ns_nhs_attn_prompt(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D,
                       int64_t cap, int64_t p0, float* out);
int ns_nhs_attn_decode_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D);
int64_t ns_nhs_attn_decode_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0);
int ns_nhs_attn_decode(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D,
                       int64_t cap, int64_t p0, float* out, float* scratch);

/* ricursive's silo names of the same two passes: heads of 128, 10 query heads a key head, ring caches [Hkv][cap][128] half
 * (slot position % cap), window win (<= 0: every key), rows Hq x 128 floats apart; _prompt more than 16 rows, _decode 1..16.
 * Replaces: kernels/llm/ricursive/silo/silo.h:38-49 (silo/attn.cpp:282-360), bound at llm/ricursive/src/ffi.rs:138-141 */
int ns_rc_flash_prompt_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D);
int ns_rc_flash_prompt(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0,
                       int64_t win, float* out);
int ns_rc_flash_decode_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D);
int64_t ns_rc_flash_decode_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0, int64_t win);
int ns_rc_flash_decode(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0,
                       int64_t win, float* out, float* scratch);

/* ---- the engines' own ("exact") attention entry points, routed to the kernels above ----------------------------- */

/* Replaces: kernels/llm/qwen35/q35.h:61-66 (q35.cpp:590-612) */
int64_t ns_q35_attn_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0);
int ns_q35_attn(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D,
                int64_t cap, int64_t p0, float* out, float* scratch);
/* Replaces: kernels/llm/museglimmer/mg.h:27-33 (mg.cpp:208-253). causal 0: the drafter's block - every row sees from
 * its own window's first key to the pass's last key; up to 16 rows it is one launch of the split kernel cut by the
 * first row's key count, longer blocks take the prompt kernel */
int64_t ns_mg_attn_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0, int64_t win, int causal);
int ns_mg_attn(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0,
               int64_t win, int causal, float* out, float* scratch);
/* The drafter's block under its silo name: ns_mg_attn with causal 0. Replaces: kernels/llm/museglimmer/silo/silo.h:53-58
 * (silo/attn.cpp:280-315); the reference covers 1..16 rows of 4 query heads a key head */
int64_t ns_mg_attn_block_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0, int64_t win);
int ns_mg_attn_block(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0,
                     int64_t win, float* out, float* scratch);
/* ricursive's attention: rows at positions p0.. against a half cache that is a ring of R rows a head (position p in slot
 * p % R); a row at position p sees the keys p - W + 1 .. p (W 0: all of 0 .. p); scale 1 / sqrt(D). D 128, 1, 2, 4, 6, 8
 * or 10 query heads a key head; the keys of a window must still be in the ring (R >= W + T - 1). Replaces:
 * kernels/llm/ricursive/rc.h:22-32 (rc.cpp:182-225), bound at llm/ricursive/src/ffi.rs:70-71 */
int ns_rc_kv_store(ns_gpu* g, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D, int64_t R, int64_t p0,
                   void* kc, void* vc);
int64_t ns_rc_attn_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t W, int64_t p0);
int ns_rc_attn(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t R,
               int64_t W, int64_t p0, float* out, float* scratch);
/* nemotron-h's attention layers: causal, no positions, scale 1 / sqrt(D), half cache [Hkv][cap][D]; D 128, query heads
 * a multiple of 8 a key head. Replaces: kernels/llm/nemotronh/nh.h:36-44 (nh.cpp:551-588), bound at
 * llm/nemotronh/src/ffi.rs:91-92 */
int ns_nh_kv_store(ns_gpu* g, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D, int64_t cap, int64_t p0,
                   void* kc, void* vc);
int64_t ns_nh_attn_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0);
int ns_nh_attn(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap,
               int64_t p0, float* out, float* scratch);
/* The weights one decode row q [Hq][D] (float32, normed and rotated) gives the n keys of a head-major cache of form kt,
 * reduced over the heads and ADDED to out [n]: their mean (mode 0) or their largest (mode 1); softmax in float32 with
 * scale 1 / sqrt(D). scratch: 2 Hq floats (each head's largest score and sum). The scores are kept [Hq][n] in memory
 * the library holds per ns_gpu (-1 when Hq x n exceeds it). D 128 or 256 (the reference: 256). Replaces:
 * kernels/llm/qwen35/q35.h:37-38 (q35.cpp:464-506), bound at llm/qwen35/src/ffi.rs:111 */
int ns_q35_attn_probs(ns_gpu* g, int kt, const float* q, const void* kc, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t n, int mode,
                      float* scratch, float* out);

/* GQA over a position-major half cache [position][G][128], q [T][H][128], explicit scale. sel NULL: dense; else
 * sel [T][G][K] names K blocks of 128 keys a (row, key head) (-1: none), cut at the row's own position (a row is a launch).
 * Replaces: kernels/llm/minimaxm3/mm3.h:33-37 (mm3.cpp:118-190). Needs scratch: this library keeps
 * ns_attn_decode_scratch(T, H, G, 128, pos0, 0) floats per ns_gpu for it (allocated at ns_gpu_open, 1 GiB) */
int ns_llm_minimaxm3_attend(ns_gpu* g, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K, float* out, int64_t T,
                            int64_t H, int64_t G, int64_t pos0, float scale);

/* The MiniMax silo's names for the same passes. Replaces: kernels/llm/minimaxm3/silo/mm3s.h:14-33,61-62 (silo/attn.cpp,
 * silo/attnx.cpp), bound at llm/minimaxm3/src/ffi.rs:164-171. One kernel family serves the vector-unit and the
 * matrix-unit names. `_split`: S = ceil(keys / 128) and part (T G S 16 130 floats) are the caller's; this library's
 * partials (splits of at least 128 keys) fit them and go there, else through the memory the library keeps per ns_gpu.
 * `_x` forms: the reference ignores `scale` and uses 1 / sqrt(128); here a positive scale is honoured, anything else
 * means 1 / sqrt(128). `_block`: a draft block, every row sees keys w0 .. pos0 + T - 1 (not causal), scale 1 / sqrt(128).
 * `_supported`: heads of 128 and H a multiple of G (the reference: H = 16 G) */
int ns_mm3s_attend_supported(int64_t H, int64_t G, int64_t head);
int ns_mm3s_attend(ns_gpu* g, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K, float* out, int64_t T, int64_t H,
                   int64_t G, int64_t pos0, float scale);
int ns_mm3s_attend_x(ns_gpu* g, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K, float* out, int64_t T, int64_t H,
                     int64_t G, int64_t pos0, float scale);
int ns_mm3s_attend_split(ns_gpu* g, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K, float* out, int64_t T,
                         int64_t H, int64_t G, int64_t pos0, float scale, int64_t S, float* part);
int ns_mm3s_attend_x_split(ns_gpu* g, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K, float* out, int64_t T,
                           int64_t H, int64_t G, int64_t pos0, float scale, int64_t S, float* part);
int ns_mm3s_attend_block(ns_gpu* g, const float* q, const uint16_t* kc, const uint16_t* vc, float* out, int64_t T, int64_t H, int64_t G, int64_t pos0,
                         int64_t w0, int64_t S, float* part);

/* kernels/llm/minimaxm3/mm3.h (indexer), mm3.cpp:59-116. The block indexer that fills `sel`: bs [T][G][nblk] = the largest
 * iq [T][G][128] . ik_j over block b's keys j <= pos0 + t (ik half [pos][128]); -inf for a block wholly past the row,
 * + 1e30 for the `local` most recent blocks. Then the K best blocks a (row, head) into sel [T][G][K], best first, the
 * lowest index of equal scores, -1 once nothing finite is left; bs is consumed (picked scores become -inf). */
int ns_llm_minimaxm3_idx_scores(ns_gpu* g, const float* iq, const uint16_t* ik, float* bs, int64_t T, int64_t G, int64_t nblk, int64_t pos0,
                                int64_t local);
int ns_llm_minimaxm3_idx_topk(ns_gpu* g, float* bs, int32_t* sel, int64_t T, int64_t G, int64_t nblk, int64_t K);

/* ---- measurement ---------------------------------------------------------------------------------------------------- */

/* This library's own (the reference times kernels from the host side: llm/qwen35/src/probe.rs:105-113). on = 1: every
 * attention call records HIP events on the compute stream before its main kernel, between it and the merge kernel, and
 * after; ns_attn_profile_last waits for the last call's and returns the two kernels' device times in nanoseconds
 * (merge_ns 0 for a call without a merge). The events open gaps between the launches and read a few microseconds long
 * for kernels this short: a kernel's own launch duration is what a kernel trace reports. on = 0 (the default): no
 * events. Every call writes its output whatever the setting; other values of `on` are refused */
int ns_attn_profile(ns_gpu* g, int on);
/* a plain device-to-device copy kernel (16 bytes a thread, reads `bytes`, writes `bytes`): the kernel of known size that
 * rocprofv3's FETCH_SIZE / WRITE_SIZE counters are scaled against. This library's own */
int ns_attn_copy_probe(ns_gpu* g, void* dst, const void* src, size_t bytes);
int ns_attn_profile_last(ns_gpu* g, double* main_ns, double* merge_ns);
/* A stretch of a pass as one submission: what is queued on g's compute stream from begin (*out: the graph) to end is
 * recorded, not run (a HIP graph by stream capture; every entry point of this library records kernel launches only);
 * end finishes it, launch replays it on g's stream, free releases it (also one still recording). A decode token recorded
 * once and replayed saves the launches' host cost and the gaps between dependent kernels.
 * Replaces: kernels/llm/qwen35/q35.h:47-52 (q35.cpp:505-549: SYCL command graphs), bound at llm/qwen35/src/ffi.rs:114-117 */
int ns_q35_graph_begin(ns_gpu* g, void** out);
int ns_q35_graph_end(ns_gpu* g, void* h);
int ns_q35_graph_launch(ns_gpu* g, void* h);
void ns_q35_graph_free(void* h);
/* Tuning knobs for sweeps and tests (this library's own): knob 0 work-groups a decode pass aims for, 1 key splits and
 * 2 waves a work-group (4 or 8) of a prompt pass, 3 work-groups an MLA pass aims for, 4 heads a wave of the
 * pre-attention kernel, 5 = 1: a prompt pass over a bfloat16, q8_0 or q4_0 cache keeps the rows' own form in the kernel
 * instead of widening them to half rows first, 5 = 2: it widens them whenever they fit; 6 the MiB of the library's own
 * scratch a pass may plan with (tests of the paths a pass takes when its rows or partials outgrow it); value 0 = the
 * library's own choice. Each knob starts from its environment variable
 * (NS_DEC_WGS, NS_PREFILL_SPLITS, NS_PREFILL_WAVES, NS_MLA_WGS, NS_PRE_HPW, NS_PREFILL_BF16, NS_SCRATCH_MIB), read once a process */
int ns_attn_tune(int knob, int64_t value);

#ifdef __cplusplus
}
#endif
#endif
