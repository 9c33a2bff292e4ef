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

// scores[h][j] = scale x sum_i q[h][i] k_j[i]: 16 lanes a key (four keys a wave), a lane D / 16 consecutive features - one
// or two 16-byte loads of a 16-bit row - the G heads in turn, each reduced over the key's 16 lanes
template <int D>
__global__ __launch_bounds__(256) void probs_scores_kernel(const float* __restrict__ q, const uint8_t* __restrict__ kc, int kt, int64_t cap, int64_t n,
                                                           int G, float scale, float* __restrict__ scores) {
    constexpr int E = D / 16;
    const int li = threadIdx.x & 15;
    const int64_t j = (int64_t) blockIdx.x * 16 + (threadIdx.x >> 4), jc = j < n ? j : n - 1;     // (whole waves reduce: a key past the end repeats the last)
    const int hk = blockIdx.y;
    const uint8_t* row = kc + ((int64_t) hk * cap + jc) * kv_row_bytes(kt, D);
    float kv[E];
    if (kt == 0 || kt == 3) {
#pragma unroll
        for (int c = 0; c < E / 8; ++c) {
            const uint4 x = *reinterpret_cast<const uint4*>(row + (li * E + c * 8) * 2);
            const uint32_t ww[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint16_t b16 = (uint16_t) (ww[e >> 1] >> (16 * (e & 1)));
                kv[c * 8 + e] = kt == 0 ? f16_to_f32(b16) : bf16_to_f32(b16);
            }
        }
    } else {
#pragma unroll
        for (int e = 0; e < E; ++e) kv[e] = kv_value_f32(row, kt, D, li * E + e);
    }
    for (int gq = 0; gq < G; ++gq) {
        const int h = hk * G + gq;
        const float4* qh = reinterpret_cast<const float4*>(q + (int64_t) h * D + li * E);
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < E / 4; ++c) {
            const float4 qv = qh[c];
            s = fmaf(qv.x, kv[c * 4], s);
            s = fmaf(qv.y, kv[c * 4 + 1], s);
            s = fmaf(qv.z, kv[c * 4 + 2], s);
            s = fmaf(qv.w, kv[c * 4 + 3], s);
        }
        s = row16_sum(s);
        if (li == 0 && j < n) scores[(int64_t) h * n + j] = s * scale;
    }
}

// a head's largest score and its sum of exp(score - largest) over a slice of the keys: part[(h nb + b) 2 ..]
__global__ __launch_bounds__(256) void probs_stats_part_kernel(const float* __restrict__ scores, int64_t n, int64_t per, float* __restrict__ part) {
    __shared__ float red[4];
    const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const float* s = scores + (int64_t) h * n;
    const int64_t j0 = (int64_t) b * per, j1 = std::min(n, j0 + per);
    float m = -INFINITY;
    for (int64_t j = j0 + tid; j < j1; j += 256) m = fmaxf(m, s[j]);
    m = wave_max(m);
    if (lane == 0) red[w] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float z = 0.0f;
    for (int64_t j = j0 + tid; j < j1; j += 256) z += expf(s[j] - m);
    z = wave_sum(z);
    if (lane == 0) red[w] = z;
    __syncthreads();
    if (tid == 0) {
        float* o = part + ((int64_t) h * gridDim.y + b) * 2;
        o[0] = m;
        o[1] = (red[0] + red[1]) + (red[2] + red[3]);
    }
}
// the slices of a head put together, in slice order: stats[2 h] the largest score, stats[2 h + 1] the sum against it
__global__ __launch_bounds__(64) void probs_stats_kernel(const float* __restrict__ part, int nb, int Hq, float* __restrict__ stats) {
    const int h = blockIdx.x * 64 + threadIdx.x;
    if (h >= Hq) return;
    const float* p = part + (int64_t) h * nb * 2;
    float m = -INFINITY;
    for (int b = 0; b < nb; ++b) m = fmaxf(m, p[2 * b]);
    float z = 0.0f;
    for (int b = 0; b < nb; ++b) z += p[2 * b + 1] * expf(p[2 * b] - m);
    stats[2 * h] = m;
    stats[2 * h + 1] = z;
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
    if ((uintptr_t) q % 16 || ((kt == 0 || kt == 3) && (uintptr_t) kc % 16)) return ns_fail("ns_q35_attn_probs: the query row and 16-bit key rows 16-byte aligned");
    // the scores, and behind them the statistics of a head's key slices (of 8192 keys and more, at most 64 a head)
    const int64_t nb = std::max<int64_t>(1, std::min<int64_t>(64, n / 8192)), per = (n + nb - 1) / nb;
    if ((size_t) (Hq * n + 2 * Hq * nb) > ns_own_floats(g)) return ns_fail("ns_q35_attn_probs: more scores (heads x keys) than the library's scratch holds");
    NS_HIP(hipSetDevice(g->dev));
    float* scores = g->own_scratch;
    float* part = scores + Hq * n;
    const float scale = 1.0f / sqrtf((float) D);
    const dim3 grid((unsigned) ((n + 15) / 16), (unsigned) Hkv);
    if (D == 128) probs_scores_kernel<128><<<grid, 256, 0, g->q>>>(q, (const uint8_t*) kc, kt, cap, n, (int) (Hq / Hkv), scale, scores);
    else probs_scores_kernel<256><<<grid, 256, 0, g->q>>>(q, (const uint8_t*) kc, kt, cap, n, (int) (Hq / Hkv), scale, scores);
    NS_LAUNCHED("probs_scores");
    probs_stats_part_kernel<<<dim3((unsigned) Hq, (unsigned) nb), 256, 0, g->q>>>(scores, n, per, part);
    NS_LAUNCHED("probs_stats_part");
    probs_stats_kernel<<<(unsigned) ((Hq + 63) / 64), 64, 0, g->q>>>(part, (int) nb, (int) Hq, scratch);
    NS_LAUNCHED("probs_stats");
    probs_out_kernel<<<(unsigned) ((n + 255) / 256), 256, 0, g->q>>>(scores, scratch, n, (int) Hq, mode, out);
    NS_LAUNCHED("probs_out");
    return 0;
    NS_CATCH
}

}  // extern "C"
