// indexer.hip: MiniMax-M3's block indexer, which feeds the block-sparse attention its lists: a score a block of 128 keys
// (the best key's), then the K best blocks a (row, key head). Bound: HBM over the indexer's half key rows (256 bytes a
// key, read once a (row, head)); selection is comparisons only and bit-exact.
//
// Reference behaviour kept: kernels/llm/minimaxm3/mm3.cpp:59-116 (scores: max over the block's keys j <= pos of iq . ik_j,
// -inf for a block wholly past the row, + 1e30 for the `local` most recent blocks; top-k: best first, the lowest index of
// equal scores, -1 once nothing finite is left, picked scores overwritten with -inf).
#include "ns_internal.hpp"
#include "ns_attn.h"
#include "kv_formats.hpp"

#include <cmath>

namespace {

constexpr int BLK = 128;

// one work-group of 128 threads a (row, head, block): a thread a key, the dot product in feature order
__global__ __launch_bounds__(BLK) void idx_scores_kernel(const float* __restrict__ iq, const uint16_t* __restrict__ ik, float* __restrict__ bs, int64_t G,
                                                         int64_t nblk, int64_t pos0, int64_t local) {
    __shared__ float qs[BLK];
    __shared__ float red[2];
    const int64_t grp = blockIdx.x;
    const int lid = threadIdx.x;
    const int64_t b = grp % nblk, tg = grp / nblk, t = tg / G;
    const int64_t pos = pos0 + t;
    qs[lid] = iq[tg * BLK + lid];
    __syncthreads();
    float v = -INFINITY;
    const int64_t j = b * BLK + lid;
    if (j <= pos) {
        const uint4* kr = reinterpret_cast<const uint4*>(ik + j * BLK);
        float s = 0.0f;
#pragma unroll 4
        for (int c = 0; c < BLK / 8; ++c) {
            const uint4 x = kr[c];
            const uint32_t ww[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
            for (int e = 0; e < 8; ++e) s += qs[c * 8 + e] * f16_to_f32((uint16_t) (ww[e >> 1] >> (16 * (e & 1))));
        }
        v = s;
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) v = fmaxf(v, __shfl_xor(v, o));
    if ((lid & 63) == 0) red[lid >> 6] = v;
    __syncthreads();
    if (lid == 0) {
        float m = fmaxf(red[0], red[1]);
        if (b * BLK > pos) m = -INFINITY;
        else if (b + local > pos / BLK) m = m + 1e30f;
        bs[grp] = m;
    }
}

// one wave a (row, head): K rounds of (largest score, its lowest index)
__global__ __launch_bounds__(64) void idx_topk_kernel(float* __restrict__ bs, int32_t* __restrict__ sel, int64_t nblk, int64_t K) {
    const int64_t row = blockIdx.x;
    const int lane = threadIdx.x;
    float* s = bs + row * nblk;
    for (int64_t k = 0; k < K; ++k) {
        float best = -INFINITY;
        for (int64_t b = lane; b < nblk; b += 64) best = fmaxf(best, s[b]);
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) best = fmaxf(best, __shfl_xor(best, o));
        int at = 0x7fffffff;
        if (best > -INFINITY)
            for (int64_t b = lane; b < nblk; b += 64)
                if (s[b] == best) { at = (int) b; break; }
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) at = min(at, __shfl_xor(at, o));
        if (lane == 0) {
            sel[row * K + k] = best > -INFINITY ? at : -1;
            if (best > -INFINITY) s[at] = -INFINITY;
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");   // the write above before the next round's reads (one wave)
        __builtin_amdgcn_s_barrier();
    }
}

}  // namespace

extern "C" {

int ns_llm_minimaxm3_idx_scores(ns_gpu* g, const float* iq, const uint16_t* ik, float* bs, int64_t T, int64_t G, int64_t nblk, int64_t pos0, int64_t local) {
    NS_TRY
    if (T <= 0 || G <= 0 || nblk <= 0) return 0;
    if (!iq || !ik || !bs) return ns_fail("ns_llm_minimaxm3_idx_scores: a null buffer");
    if ((uintptr_t) ik % 16) return ns_fail("ns_llm_minimaxm3_idx_scores: key rows 16-byte aligned");
    if (T * G * nblk > (int64_t) 1 << 31) return ns_fail("ns_llm_minimaxm3_idx_scores: too many blocks");
    NS_HIP(hipSetDevice(g->dev));
    idx_scores_kernel<<<(unsigned) (T * G * nblk), BLK, 0, g->q>>>(iq, ik, bs, G, nblk, pos0, local);
    NS_LAUNCHED("idx_scores");
    return 0;
    NS_CATCH
}

int ns_llm_minimaxm3_idx_topk(ns_gpu* g, float* bs, int32_t* sel, int64_t T, int64_t G, int64_t nblk, int64_t K) {
    NS_TRY
    if (T <= 0 || G <= 0 || K <= 0) return 0;
    if (nblk < 0) return ns_fail("ns_llm_minimaxm3_idx_topk: a block count");
    if (!bs || !sel) return ns_fail("ns_llm_minimaxm3_idx_topk: a null buffer");
    NS_HIP(hipSetDevice(g->dev));
    idx_topk_kernel<<<(unsigned) (T * G), 64, 0, g->q>>>(bs, sel, nblk, K);
    NS_LAUNCHED("idx_topk");
    return 0;
    NS_CATCH
}

}  // extern "C"
