/* ns_mla.h - multi-head latent attention (DeepSeek-V3 / R1's absorbed form, GLM-5.3's latent-only form) of
 * libnextsycl-llm.so on one AMD MI355X (gfx950). Conventions as ns_attn.h: everything queued on the ns_gpu's compute
 * stream, 0 or -1 with the reason in ns_last_error(), the caller owns every buffer.
 *
 * The latent cache (reference: kernels/llm/deepseek2/ds2.h:28-31): one row a position, shared by all heads,
 *   DeepSeek   [512 latent | 64 rope-rotated key] half         1152 bytes
 *   GLM        [512 latent] half                               1024 bytes
 *   GLM q8     [16 half scales][512 int8]                       544 bytes   (kernels/llm/glm5next/glm.cpp:1074-1077)
 * Row t of a pass sits at position pos0 + t and reads cells 0 .. pos0 + t.
 */
#ifndef NS_MLA_H
#define NS_MLA_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ns_gpu ns_gpu;

/* The absorbed decode up to the latent sum (BASELINE's MLA configuration ends here): qa [T][H][512 + R] already absorbed
 * and rotated ([k_b q_nope | q_pe]), element type qt (0 float32, 1 half); cache rows [512 + R] half; u [T][H][512] of
 * type qt = softmax_i(scale qa . c_i) c_i[:512], row t over cells 0 .. pos0 + t. R 64 or 0. T 1..16 is a decode or
 * verify pass; a prompt's rows (any T) run 16 a pass on the queue. `scratch`: ns_mla_decode_latent_scratch floats.
 * This library's own entry point: the reference computes u inside ns_ds2_mla_decode / ns_mla_attend_sel at decode
 * widths and, for prompts and contexts past 8192 cells, as a chain of half GEMMs and a masked softmax over the same
 * rows (llm/deepseek2/src/engine.rs:1165-1253; kernels/llm/glm5next/glm.cpp:208-277, 1042-1060) */
int64_t ns_mla_decode_latent_scratch(int64_t T, int64_t H, int64_t pos0);
int ns_mla_decode_latent(ns_gpu* g, int qt, const void* qa, const uint16_t* cache, void* u, int64_t T, int64_t H, int64_t R, int64_t pos0,
                         float scale, float* scratch);

/* MLA at decode widths in one call: q [T][H][128 nope + 64 rope] (rope part rotated), k_b [H][512][128] and v_b
 * [H][128][512] half, cache [n][576] half -> out [T][H][128] = v_b u. Runs absorb, the latent decode and the value
 * up-projection; its scratch is the library's own (kept per ns_gpu, 1 GiB). Replaces:
 * kernels/llm/deepseek2/ds2.h:32-37 (ds2.cpp:139-258, 262-270) */
int ns_ds2_mla_decode(ns_gpu* g, const float* q, const uint16_t* kb, const uint16_t* vb, const uint16_t* cache, float* out, int64_t T, int64_t H,
                      int64_t pos0, float scale);
/* The same with kv_b as the model file stores it - Q6_K, [H x (nope + V)] rows of L = 512 (two 210-byte blocks a row): per
 * head its 128 k rows (k_i[c]: q~[c] = sum_i q_nope[i] k_i[c]), then its 128 v rows - decoded where it is read. Replaces:
 * kernels/llm/deepseek2/ds2.h:38-41 (ds2.cpp:117-134,157-173,237-246,272-281) */
int ns_ds2_mla_decode_q6k(ns_gpu* g, const float* q, const void* kvb, const uint16_t* cache, float* out, int64_t T, int64_t H, int64_t pos0,
                          float scale);
/* ggml's YaRN rope (adjacent pairs) in place on x: T rows `row` floats apart, H heads `head` floats apart, the rotated
 * part n_dims values from float `off` of each head, row t at position pos0 + t; out (nullable): the rotated part also
 * written there (rows out_row, heads out_head floats apart). The decode step's q_pe (and k_pe, where an engine keeps it
 * apart from the latent cache). Replaces: kernels/llm/deepseek2/ds2.h:20-27 (ds2.cpp:59-83) */
int ns_ds2_rope(ns_gpu* g, float* x, int64_t T, int64_t H, int64_t row, int64_t head, int64_t off, int64_t n_dims, int64_t pos0,
                float freq_base, float freq_scale, float ext_factor, float mscale, float corr0, float corr1, float* out, int64_t out_row,
                int64_t out_head);
/* The latent cache's rows pos0 .. pos0 + T - 1 from kv [T][L + R] float32: the first L RMS-normed with w (eps), the last
 * R rotated by ggml's YaRN rope on adjacent pairs. Replaces: kernels/llm/deepseek2/ds2.h:28-31 (ds2.cpp:85-112) */
int ns_ds2_kv_store(ns_gpu* g, const float* kv, const float* w, float eps, uint16_t* cache, int64_t T, int64_t L, int64_t R, int64_t pos0,
                    float freq_base, float freq_scale, float ext_factor, float mscale, float corr0, float corr1);

/* GLM-5.3's latent-only MLA over a half cache [n][512]: qa [T][H][512] float32 -> u [T][H][512] float32. sel_cnt NULL:
 * every row sees every earlier cell. Else row t's cells are the pools sel[t K ..][0, sel_cnt[t]) of 4 cells each (cells
 * 4 b .. 4 b + 3) followed by its incomplete pool 4 ((p + 1) / 4) .. p, p = pos0 + t; a negative sel_cnt[t] is a dense
 * row. Any number of rows: rows with lists go 16 a pass on the queue, dense
 * rows as a prompt's. L = 512, or 256 (cache [n][256], qa and u [T][H][256]: the same kernel built for rows half as wide).
 * Replaces: kernels/llm/glm5next/glm.h:65-66 (glm.cpp:1062-1067,1095-1102,1252-1264) */
int ns_mla_attend_sel(ns_gpu* g, const float* qa, const uint16_t* c, float* u, int64_t T, int64_t H, int64_t L, int64_t pos0, float scale,
                      const int32_t* sel, const int32_t* sel_cnt, int64_t K);
/* the same over q8 latent rows. Replaces: kernels/llm/glm5next/glm.h:79-80 (glm.cpp:1267-1276; the reference: at most 8 rows) */
int ns_mla_attend_sel_q8(ns_gpu* g, const float* qa, const void* c, float* u, int64_t T, int64_t H, int64_t L, int64_t pos0, float scale,
                         const int32_t* sel, const int32_t* sel_cnt, int64_t K);
/* The dense form over a float32 latent cache c [n][L], L = 512 or 256 (every row sees every earlier cell): the cells
 * 0 .. pos0 + T - 1 are rounded to half into memory the library keeps per ns_gpu and read from there (-1 when they do not
 * fit beside the partials: ~200,000 cells of 512). Replaces: kernels/llm/glm5next/glm.h:47 (glm.cpp:782-812) */
int ns_mla_attend(ns_gpu* g, const float* qa, const float* c, float* u, int64_t T, int64_t H, int64_t L, int64_t pos0, float scale);
/* GLM's DSA indexer, which fills the lists ns_mla_attend_sel reads (pools of 4 consecutive tokens). Replaces:
 * kernels/llm/glm5next/glm.h:48-55 (glm.cpp:876-1019), bound at llm/glm5next/src/ffi.rs.
 * ns_idx_pool: the pools completed by tokens [pos0, pos0 + T): pooled[j][c] = sum_m softmax_m(ig_m[c] + ape[m][c]) ik_m[c]
 *   over pool j's 4 members (ik, ig [T][D] float32, ape [4][D]); a member before pos0 comes from ring [8][2 D] (ik | ig at
 *   slot position % 8), which then takes this pass's last (up to 8) tokens.
 * ns_idx_score: S [T H][n] (iq . pooled^T for pools [j0, j0 + n), the engine's GEMM), w [T][H]: score[r][j0 + jj] =
 *   sum_h max(S[r H + h][jj], 0) w[r][h], heads in order, for the pools row r sees (j < (pos0 + r + 1) / 4), else -inf;
 *   score rows ld floats apart.
 * ns_topk: the K highest of score[r][0, n) into sel[r][0, K) as positions in ascending order, ties at the K-th value to the
 *   lowest positions; the same list every run. */
int ns_idx_pool(ns_gpu* g, float* ring, const float* ik, const float* ig, const float* ape, float* pooled, int64_t pos0, int64_t T, int64_t D);
int ns_idx_score(ns_gpu* g, const float* S, const float* w, float* score, int64_t T, int64_t H, int64_t j0, int64_t n, int64_t ld, int64_t pos0);
int ns_topk(ns_gpu* g, const float* score, int32_t* sel, int64_t T, int64_t n, int64_t ld, int64_t K);
/* The pieces of the reference's prompt path around its GEMMs (ns_mla_attend_sel with any T does the whole of that path
 * in one call; these serve an engine that keeps the reference's chain). Replaces: kernels/llm/glm5next/glm.h:58-60
 * (glm.cpp:1023-1060), bound at llm/glm5next/src/ffi.rs:117.
 * ns_mla_cells: each row's cells as a list - idx [T][NC] int32 (0 past the row's cells), n [T] their count, at most NC:
 *   with lists (sel [T][K], sel_cnt [T]) the 4 tokens of each listed pool, then the row's incomplete pool; sel_cnt null
 *   or sel_cnt[t] < 0: every cell up to the row's own position pos0 + t.
 * ns_softmax_masked: S [R H][NC] in place: softmax of scale x S over the first n[r] cells of row r's H heads, 0 behind. */
int ns_mla_cells(ns_gpu* g, const int32_t* sel, const int32_t* sel_cnt, int64_t T, int64_t K, int64_t pos0, int32_t* idx, int32_t* n, int64_t NC);
int ns_softmax_masked(ns_gpu* g, float* S, int64_t R, int64_t H, int64_t NC, const int32_t* n, float scale);
/* out [n][512] half = the q8 latent rows idx[i] of src, widened: half(scale x q), one rounding (a prompt pass's gather).
 * Replaces: kernels/llm/glm5next/glm.h:78 (glm.cpp:1301-1325) */
int ns_gather_q8_h(ns_gpu* g, const void* src, const int32_t* idx, uint16_t* out, int64_t n, int64_t L);
/* rows x [n][512] float32 -> q8 latent rows y [n][544]: a block's scale amax / 127 rounded to half BEFORE the values are
 * divided by it, round half away from zero, clamp to +-127. Replaces: kernels/llm/glm5next/glm.h:77 (glm.cpp:1282-1299) */
int ns_to_q8row(ns_gpu* g, const float* x, void* y, int64_t n, int64_t L);
/* The half products of that chain (the reference: oneMKL). y [T, N] (+)= x [T, K] . w [N, K]^T, x and w half, y and the
 * sums float32; rows of x ldx, of y ldy elements apart, accumulate != 0 adds to y. ns_gemm_batch_h: `batch` such
 * products, operand b at x + b sx, w + b sw, y + b sy (elements); op(w) = w^T (w [N, K], rows ldw apart) with trans_w,
 * else w ([K, N]). Any sizes and strides; 16-byte aligned operands with strides in multiples of 8 load fastest.
 * ns_to_f16: y[i] = half(x[i]), round to nearest even. Replaces: kernels/llm/glm5next/glm.h:81-82 (glm.cpp:217-225),
 * glm.h:63-64 (glm.cpp:265-276), glm.h:73 (glm.cpp:208-214), bound at llm/glm5next/src/ffi.rs */
int ns_gemm_f16(ns_gpu* g, int64_t T, int64_t N, int64_t K, const uint16_t* x, int64_t ldx, const uint16_t* w, float* y, int64_t ldy,
                int accumulate);
int ns_gemm_batch_h(ns_gpu* g, int64_t batch, int trans_w, int64_t T, int64_t N, int64_t K, const uint16_t* x, int64_t ldx, int64_t sx,
                    const uint16_t* w, int64_t ldw, int64_t sw, float* y, int64_t ldy, int64_t sy, int accumulate);
int ns_to_f16(ns_gpu* g, const float* x, uint16_t* y, int64_t n);
/* out [n][C] half = the rows idx[i] of src (rows of C halfs, C a multiple of 8): the cells of a prompt pass's rows gathered
 * out of a half latent cache, as ns_gather_q8_h does out of a q8 one. Replaces: kernels/llm/glm5next/glm.h:75
 * (glm.cpp:842-853), called at llm/glm5next/src/engine.rs:106-108,1925 */
int ns_gather_h(ns_gpu* g, const uint16_t* src, const int32_t* idx, uint16_t* out, int64_t n, int64_t C);

#ifdef __cplusplus
}
#endif
#endif
