// attn_probs.hip: the attention weights one decode row gives every key, reduced over the heads (gfx950).
//
// The engine's attention capture (llm/qwen35/src/engine.rs:1468-1487) asks, for a one-row pass, how much weight each of
// the n cached positions received: out[j] += mean_h p_h(j) (mode 0) or max_h p_h(j) (mode 1), p_h = softmax_j(q_h . k_j /
// sqrt(D)) in float32 over the cache's keys as the attention kernels read them into float32. Reference:
// kernels/llm/qwen35/q35.cpp:464-506 - three sweeps that recompute every score. Here the scores are computed once (a
// wave a key, the key's row read once for the G query heads that share it) and kept [Hq][n] in the library's scratch.
//
// Bound: HBM, n x row bytes read once; a diagnostic call, not on the decode path's critical path.
#include "ns_internal.hpp"
#include "ns_attn.h"
#include "attn_common.hpp"
#include "attn_host.hpp"
#include "kv_formats.hpp"

#include <cmath>

namespace {

// scores[h][j] = scale x sum_i q[h][i] k_j[i]: a wave a key, a lane D / 64 consecutive features, the G heads in turn
template <int D>
__global__ __launch_bounds__(256) void probs_scores_kernel(const float* __restrict__ q, const uint8_t* __restrict__ kc, int kt, int64_t cap, int64_t n,
                                                           int G, float scale, float* __restrict__ scores) {
    constexpr int E = D / 64;
    const int lane = threadIdx.x & 63;
    const int64_t j = (int64_t) blockIdx.x * 4 + (threadIdx.x >> 6);
    const int hk = blockIdx.y;
    if (j >= n) return;
    const uint8_t* row = kc + ((int64_t) hk * cap + j) * kv_row_bytes(kt, D);
    float kv[E];
#pragma unroll
    for (int e = 0; e < E; ++e) kv[e] = kv_value_f32(row, kt, D, lane * E + e);
    for (int gq = 0; gq < G; ++gq) {
        const int h = hk * G + gq;
        const float* qh = q + (int64_t) h * D + lane * E;
        float s = 0.0f;
#pragma unroll
        for (int e = 0; e < E; ++e) s = fmaf(qh[e], kv[e], s);
        s = wave_sum(s);
        if (lane == 0) scores[(int64_t) h * n + j] = s * scale;
    }
}

// a head's largest score and the sum of exp(score - largest): stats[2 h], stats[2 h + 1]
__global__ __launch_bounds__(256) void probs_stats_kernel(const float* __restrict__ scores, int64_t n, float* __restrict__ stats) {
    __shared__ float red[4];
    const int h = blockIdx.x, tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const float* s = scores + (int64_t) h * n;
    float m = -INFINITY;
    for (int64_t j = tid; j < n; j += 256) m = fmaxf(m, s[j]);
    m = wave_max(m);
    if (lane == 0) red[w] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float z = 0.0f;
    for (int64_t j = tid; j < n; j += 256) z += expf(s[j] - m);
    z = wave_sum(z);
    if (lane == 0) red[w] = z;
    __syncthreads();
    if (tid == 0) {
        stats[2 * h] = m;
        stats[2 * h + 1] = (red[0] + red[1]) + (red[2] + red[3]);
    }
}

// out[j] += the heads' weights of key j: their mean (mode 0) or their largest (mode 1)
__global__ __launch_bounds__(256) void probs_out_kernel(const float* __restrict__ scores, const float* __restrict__ stats, int64_t n, int Hq, int mode,
                                                        float* __restrict__ out) {
    const int64_t j = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (j >= n) return;
    float acc = 0.0f;
    for (int h = 0; h < Hq; ++h) {
        const float p = expf(scores[(int64_t) h * n + j] - stats[2 * h]) / stats[2 * h + 1];
        acc = mode == 1 ? fmaxf(acc, p) : acc + p / (float) Hq;
    }
    out[j] += acc;
}

}  // namespace

extern "C" {

int ns_q35_attn_probs(ns_gpu* g, int kt, const float* q, const void* kc, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t n, int mode,
                      float* scratch, float* out) {
    NS_TRY
    if (n <= 0) return 0;
    if (n > cap || Hkv <= 0 || Hq <= 0 || Hq % Hkv || (D != 128 && D != 256) || kt < 0 || kt > 3)
        return ns_fail("ns_q35_attn_probs: keys past the cache, heads that do not share, or not heads of 128 or 256");
    if (!q || !kc || !scratch || !out) return ns_fail("ns_q35_attn_probs: a null buffer");
    if (Hkv > 65535) return ns_fail("ns_q35_attn_probs: at most 65535 key heads");
    if ((size_t) (Hq * n) > ns_own_floats(g)) return ns_fail("ns_q35_attn_probs: more scores (heads x keys) than the library's scratch holds");
    NS_HIP(hipSetDevice(g->dev));
    float* scores = g->own_scratch;
    const float scale = 1.0f / sqrtf((float) D);
    const dim3 grid((unsigned) ((n + 3) / 4), (unsigned) Hkv);
    if (D == 128) probs_scores_kernel<128><<<grid, 256, 0, g->q>>>(q, (const uint8_t*) kc, kt, cap, n, (int) (Hq / Hkv), scale, scores);
    else probs_scores_kernel<256><<<grid, 256, 0, g->q>>>(q, (const uint8_t*) kc, kt, cap, n, (int) (Hq / Hkv), scale, scores);
    NS_LAUNCHED("probs_scores");
    probs_stats_kernel<<<(unsigned) Hq, 256, 0, g->q>>>(scores, n, scratch);
    NS_LAUNCHED("probs_stats");
    probs_out_kernel<<<(unsigned) ((n + 255) / 256), 256, 0, g->q>>>(scores, scratch, n, (int) Hq, mode, out);
    NS_LAUNCHED("probs_out");
    return 0;
    NS_CATCH
}

}  // extern "C"
