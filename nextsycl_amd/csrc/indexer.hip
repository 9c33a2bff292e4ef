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
#include "attn_common.hpp"

#include <algorithm>
#include <cmath>

namespace {

constexpr int BLK = 128;

// one work-group of 128 threads a block of 128 keys: a thread holds its key's row (read once, whatever the number of
// rows and heads) and takes its dot product - in feature order - with every (row, head) query in turn; the block's best
// a query is reduced over the two waves
constexpr int QCH = 16;     // queries staged in LDS at a time

__global__ __launch_bounds__(BLK) void idx_scores_kernel(const float* __restrict__ iq, const uint16_t* __restrict__ ik, float* __restrict__ bs, int64_t TG,
                                                         int64_t G, int64_t nblk, int64_t pos0, int64_t local) {
    __shared__ float qs[QCH][BLK];
    __shared__ float red[QCH][2];
    const int64_t b = blockIdx.x;
    const int lid = threadIdx.x;
    const int64_t j = b * BLK + lid, last = pos0 + (TG - 1) / G;      // the pass's last row sees the most keys
    float kf[BLK];              // the key's row widened once: 128 registers
    {
        uint4 row[BLK / 8];
        const uint4* kr = reinterpret_cast<const uint4*>(ik + std::min(j, last) * BLK);
#pragma unroll
        for (int c = 0; c < BLK / 8; ++c) row[c] = kr[c];
#pragma unroll
        for (int c = 0; c < BLK / 8; ++c) {
            const uint32_t ww[4] = {row[c].x, row[c].y, row[c].z, row[c].w};
#pragma unroll
            for (int e = 0; e < 8; ++e) kf[c * 8 + e] = f16_to_f32((uint16_t) (ww[e >> 1] >> (16 * (e & 1))));
        }
    }
    for (int64_t q0 = 0; q0 < TG; q0 += QCH) {
        const int nq = (int) std::min<int64_t>(QCH, TG - q0);
        __syncthreads();
        for (int i = 0; i < nq; ++i) qs[i][lid] = iq[(q0 + i) * BLK + lid];
        __syncthreads();
        for (int i = 0; i < nq; ++i) {
            const int64_t pos = pos0 + (q0 + i) / G;
            float s = 0.0f;
#pragma unroll
            for (int d = 0; d < BLK; ++d) s += qs[i][d] * kf[d];
            const float v = wave_max(j <= pos ? s : -INFINITY);
            if ((lid & 63) == 0) red[i][lid >> 6] = v;
        }
        __syncthreads();
        if (lid < nq) {
            const int64_t pos = pos0 + (q0 + lid) / G;
            float m = fmaxf(red[lid][0], red[lid][1]);
            if (b * BLK > pos) m = -INFINITY;
            else if (b + local > pos / BLK) m = m + 1e30f;
            bs[(q0 + lid) * nblk + b] = m;
        }
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

// the same selection with the row's scores held in registers (VPL a lane: rows of up to 64 VPL blocks): a round is a
// few compares and two wave reductions instead of two passes over the row in memory and a fence. The chosen blocks'
// scores are overwritten with -inf in memory too, as the kernel above leaves them.
template <int VPL>
__global__ __launch_bounds__(64) void idx_topk_reg_kernel(float* __restrict__ bs, int32_t* __restrict__ sel, int nblk, int K) {
    const int64_t row = blockIdx.x;
    const int lane = threadIdx.x;
    float* s = bs + row * nblk;
    float v[VPL];
#pragma unroll
    for (int j = 0; j < VPL; ++j) v[j] = lane + 64 * j < nblk ? s[lane + 64 * j] : -INFINITY;
    for (int k = 0; k < K; ++k) {
        float best = -INFINITY;
#pragma unroll
        for (int j = 0; j < VPL; ++j) best = fmaxf(best, v[j]);
        best = wave_max(best);
        int at = 0x7fffffff;
        if (best > -INFINITY) {
#pragma unroll
            for (int j = VPL - 1; j >= 0; --j) at = v[j] == best ? lane + 64 * j : at;     // this lane's lowest index of it
        }
        at = wave_min(at);
        if (best > -INFINITY) {
#pragma unroll
            for (int j = 0; j < VPL; ++j)
                if (lane + 64 * j == at) {
                    v[j] = -INFINITY;
                    s[at] = -INFINITY;
                }
        }
        if (lane == 0) sel[row * K + k] = best > -INFINITY ? at : -1;
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
    idx_scores_kernel<<<(unsigned) nblk, BLK, 0, g->q>>>(iq, ik, bs, T * G, G, nblk, pos0, local);
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
    const unsigned rows = (unsigned) (T * G);
    if (K > (int64_t) 1 << 30) return ns_fail("ns_llm_minimaxm3_idx_topk: a list length");
    if (nblk <= 64 * 8) idx_topk_reg_kernel<8><<<rows, 64, 0, g->q>>>(bs, sel, (int) nblk, (int) K);
    else if (nblk <= 64 * 32) idx_topk_reg_kernel<32><<<rows, 64, 0, g->q>>>(bs, sel, (int) nblk, (int) K);
    else if (nblk <= 64 * 128) idx_topk_reg_kernel<128><<<rows, 64, 0, g->q>>>(bs, sel, (int) nblk, (int) K);
    else idx_topk_kernel<<<rows, 64, 0, g->q>>>(bs, sel, nblk, K);
    NS_LAUNCHED("idx_topk");
    return 0;
    NS_CATCH
}

}  // extern "C"
