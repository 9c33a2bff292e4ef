// indexer.hip: MiniMax-M3's block indexer, which feeds the block-sparse attention its lists: a score a block of 128 keys
// (the best key's), then the K best blocks a (row, key head). Bound: HBM over the indexer's half key rows (256 bytes a
// key, read once a (row, head)); selection is comparisons only and bit-exact.
//
// Reference behaviour kept: kernels/llm/minimaxm3/mm3.cpp:59-116 (scores: max over the block's keys j <= pos of iq . ik_j,
// -inf for a block wholly past the row, + 1e30 for the `local` most recent blocks; top-k: best first, the lowest index of
// equal scores, -1 once nothing finite is left, picked scores overwritten with -inf).
#include "ns_internal.hpp"
#include "ns_attn.h"
#include "ns_mla.h"
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

// (a prompt's thousands of queries are dealt to grid.y slices of qper queries each: a work-group is two waves, and one
// a key block - 272 of them behind 32768 keys - left three SIMDs in four idle: 2048 rows x 4 heads 6.5 ms)
__global__ __launch_bounds__(BLK) void idx_scores_kernel(const float* __restrict__ iq, const uint16_t* __restrict__ ik, float* __restrict__ bs, int64_t TG,
                                                         int64_t G, int64_t nblk, int64_t pos0, int64_t local, int64_t qper) {
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
    const int64_t qbeg = (int64_t) blockIdx.y * qper, qend = std::min(TG, qbeg + qper);
    for (int64_t q0 = qbeg; q0 < qend; q0 += QCH) {
        const int nq = (int) std::min<int64_t>(QCH, qend - q0);
        __syncthreads();
        for (int i = 0; i < nq; ++i) qs[i][lid] = iq[(q0 + i) * BLK + lid];
        __syncthreads();
        for (int i = 0; i < nq; ++i) {
            const int64_t pos = pos0 + (q0 + i) / G;
            // (the query's features as scalar operands straight from memory instead - they are the same for every lane -
            // were measured twice as slow: every multiply-add then waits for the scalar load in front of it)
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

// ---- GLM's DSA indexer (kernels/llm/glm5next/glm.cpp:876-1019): pools of 4 consecutive tokens --------------------------

// the pools completed by this pass: pooled[j][c] = sum_m softmax_m(ig_m[c] + ape[m][c]) ik_m[c] over pool j's 4 members
// (positions 4 j + m; a member before pos0 comes from the ring: ik | ig at slot position % 8). A thread a (pool, feature)
__global__ __launch_bounds__(256) void glm_idx_pool_kernel(const float* __restrict__ ring, const float* __restrict__ ik, const float* __restrict__ ig,
                                                           const float* __restrict__ ape, float* __restrict__ pooled, int64_t pos0, int64_t j_lo, int64_t npool,
                                                           int64_t D) {
    const int64_t gi = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (gi >= npool * D) return;
    const int64_t j = j_lo + gi / D, c = gi % D;
    float lg[4], kv[4], mx = -INFINITY;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        const int64_t pp = 4 * j + m;
        const float* k = pp >= pos0 ? ik + (pp - pos0) * D : ring + (pp % 8) * 2 * D;
        const float* gg = pp >= pos0 ? ig + (pp - pos0) * D : ring + (pp % 8) * 2 * D + D;
        kv[m] = k[c];
        lg[m] = gg[c] + ape[m * D + c];
        mx = fmaxf(mx, lg[m]);
    }
    float sum = 0.0f, acc = 0.0f;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        const float e = expf(lg[m] - mx);
        sum += e;
        acc += e * kv[m];
    }
    pooled[j * D + c] = acc / sum;
}

// the ring takes the pass's last (up to 8) tokens: ik | ig at slot position % 8
__global__ __launch_bounds__(256) void glm_idx_ring_kernel(float* __restrict__ ring, const float* __restrict__ ik, const float* __restrict__ ig, int64_t pos0,
                                                           int64_t first, int64_t rows, int64_t D) {
    const int64_t gi = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (gi >= rows * D) return;
    const int64_t pp = first + gi / D, c = gi % D;
    ring[(pp % 8) * 2 * D + c] = ik[(pp - pos0) * D + c];
    ring[(pp % 8) * 2 * D + D + c] = ig[(pp - pos0) * D + c];
}

// score[r][j0 + jj] = sum_h relu(S[r H + h][jj]) w[r][h] in head order for the pools row r sees, -inf for the others
__global__ __launch_bounds__(256) void glm_idx_score_kernel(const float* __restrict__ S, const float* __restrict__ w, float* __restrict__ score, int64_t T,
                                                            int64_t H, int64_t j0, int64_t n, int64_t ld, int64_t pos0) {
    const int64_t gi = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (gi >= T * n) return;
    const int64_t r = gi / n, jj = gi % n, j = j0 + jj;
    const int64_t nv = (pos0 + r + 1) / 4;
    float s = -INFINITY;
    if (j < nv) {
        s = 0.0f;
        for (int64_t h = 0; h < H; ++h) s += fmaxf(S[(r * H + h) * n + jj], 0.0f) * w[r * H + h];
    }
    score[r * ld + j] = s;
}

// the K highest of a row's n scores as positions in ascending order, ties at the K-th value to the lowest positions: a
// radix select over the floats' order-preserving keys (4 digits of 8 bits, a histogram a digit in LDS), then one ordered
// compaction - every thread its own run of positions, two scans over the work-group, no atomics in what is written, so
// the list (and the sums of the attention that reads it) is the same every run. A work-group of 1024 a row.
constexpr int TOPK_WG = 1024, TOPK_NH = 16;
__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = __builtin_bit_cast(uint32_t, f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);             // a larger float, a larger key
}
// exclusive prefix sum of one value a thread over the work-group (the total to every thread through `total`)
__device__ uint32_t wg_exclusive_scan(uint32_t v, uint32_t* wsum, uint32_t& total) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    uint32_t x = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const uint32_t y = __shfl_up(x, o, 64);
        if (lane >= o) x += y;
    }
    if (lane == 63) wsum[wv] = x;
    __syncthreads();
    uint32_t before = 0, all = 0;
    for (int i = 0; i < TOPK_WG / 64; ++i) {
        const uint32_t t = wsum[i];
        if (i < wv) before += t;
        all += t;
    }
    __syncthreads();
    total = all;
    return before + x - v;
}
__global__ __launch_bounds__(TOPK_WG) void glm_topk_kernel(const float* __restrict__ score, int32_t* __restrict__ sel, int64_t n, int64_t ld, int64_t K) {
    __shared__ uint32_t hist[TOPK_NH * 256];
    __shared__ uint32_t st[3];                                     // prefix, mask, still needed
    __shared__ uint32_t wsum[TOPK_WG / 64];
    const int64_t r = blockIdx.x;
    const int lid = threadIdx.x;
    const float* row = score + r * ld;
    if (lid == 0) {
        st[0] = 0;
        st[1] = 0;
        st[2] = (uint32_t) K;
    }
    uint32_t* mine = hist + (lid % TOPK_NH) * 256;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int b = lid; b < TOPK_NH * 256; b += TOPK_WG) hist[b] = 0;
        __syncthreads();
        const uint32_t prefix = st[0], mask = st[1];
        for (int64_t j = lid; j < n; j += TOPK_WG) {
            const uint32_t k = order_key(row[j]);
            if ((k & mask) == prefix) atomicAdd(&mine[(k >> shift) & 255], 1u);
        }
        __syncthreads();
        if (lid < 256) {
            uint32_t c = 0;
            for (int m = 0; m < TOPK_NH; ++m) c += hist[m * 256 + lid];
            hist[lid] = c;
        }
        __syncthreads();
        if (lid == 0) {
            // the digit, from the top, at which the count of keys at or above it reaches what is still needed
            const uint32_t need = st[2];
            uint32_t above = 0;
            int d = 255;
            for (; d > 0; --d) {
                if (above + hist[d] >= need) break;
                above += hist[d];
            }
            st[0] = prefix | ((uint32_t) d << shift);
            st[1] = mask | (255u << shift);
            st[2] = need - above;
        }
        __syncthreads();
    }
    const uint32_t kth = st[0], ties = st[2];
    const int64_t seg = (n + TOPK_WG - 1) / TOPK_WG, j0 = std::min<int64_t>(n, lid * seg), j1 = std::min<int64_t>(n, j0 + seg);
    uint32_t gt = 0, eq = 0;
    for (int64_t j = j0; j < j1; ++j) {
        const uint32_t k = order_key(row[j]);
        gt += k > kth;
        eq += k == kth;
    }
    uint32_t total;
    const uint32_t eq_before = wg_exclusive_scan(eq, wsum, total);
    const uint32_t eq_take = eq_before >= ties ? 0u : std::min(eq, ties - eq_before);
    uint32_t at = wg_exclusive_scan(gt + eq_take, wsum, total);
    uint32_t eq_left = eq_take;
    for (int64_t j = j0; j < j1; ++j) {
        const uint32_t k = order_key(row[j]);
        if (k > kth || (k == kth && eq_left > 0)) {
            if (k == kth) --eq_left;
            if (at < (uint32_t) K) sel[r * K + at] = (int32_t) j;
            ++at;
        }
    }
}

// The same selection for rows of up to PER x 1024 scores, their keys held in registers (score j = i 1024 + lid: loaded
// once, coalesced, all in flight) - the row is read from memory once instead of five times with a dependent load an
// iteration. The histogram has a copy a lane (64 copies, 257 words apart: the lanes of a wave never meet in an address or
// a bank, however few digits the row's scores share - the top digit, sign and exponent, takes a handful of values), the
// digit is found by a suffix scan over 256 threads instead of one thread's walk, and a position's place in the list = the
// greater keys before it + the equal ones before it that are still taken, both from ballots and one scan (below).
template <int PER>
__global__ __launch_bounds__(TOPK_WG) void glm_topk_reg_kernel(const float* __restrict__ score, int32_t* __restrict__ sel, int n, int64_t ld, int K) {
    constexpr int NC = 64, CS = 257;
    __shared__ uint32_t hist[NC * CS];
    __shared__ uint32_t st[3];
    __shared__ uint32_t wsum[TOPK_WG / 64];
    const int64_t r = blockIdx.x;
    const int lid = threadIdx.x, lane = lid & 63, wv = lid >> 6;
    const float* row = score + r * ld;
    uint32_t key[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = i * TOPK_WG + lid;
        key[i] = j < n ? order_key(row[j]) : 0u;
    }
    if (lid == 0) {
        st[0] = 0;
        st[1] = 0;
        st[2] = (uint32_t) K;
    }
    uint32_t* mine = hist + lane * CS;
    for (int shift = 24; shift >= 0; shift -= 8) {
        for (int b = lid; b < NC * CS; b += TOPK_WG) hist[b] = 0;
        __syncthreads();
        const uint32_t prefix = st[0], mask = st[1], need = st[2];
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int j = i * TOPK_WG + lid;
            if (j < n && (key[i] & mask) == prefix) atomicAdd(&mine[(key[i] >> shift) & 255], 1u);
        }
        __syncthreads();
        // thread lid < 256 takes digit d = 255 - lid: its count, then the count of every digit at or above it
        uint32_t c = 0, incl = 0;
        const int d = 255 - lid;
        if (lid < 256) {
            for (int m = 0; m < NC; ++m) c += hist[m * CS + d];
            incl = c;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const uint32_t y = __shfl_up(incl, o, 64);
                if (lane >= o) incl += y;
            }
            if (lane == 63) wsum[wv] = incl;
        }
        __syncthreads();
        if (lid < 256) {
            for (int x = 0; x < wv; ++x) incl += wsum[x];
            const uint32_t above = incl - c;                       // keys in digits above d
            if (above < need && (incl >= need || d == 0)) {        // (d = 0 takes what is left, as the walk from the top does)
                st[0] = prefix | ((uint32_t) d << shift);
                st[1] = mask | (255u << shift);
                st[2] = need - above;
            }
        }
        __syncthreads();
    }
    // The list in position order: position j = i 1024 + 64 wv + lane. Every wave counts its greater and its equal keys a
    // slice i (two ballots), the counts' running sums over (slice, wave) - 16 PER entries in that order - are one
    // work-group scan each, and a key's place is then its wave's running sum plus the lanes before it in its ballot.
    const uint32_t kth = st[0], ties = st[2];
    uint32_t* const cg = hist;                                     // [PER][16] greater keys a (slice, wave), then their running sums
    uint32_t* const ce = hist + PER * 16;                          // the same for the equal keys
    constexpr int NW = TOPK_WG / 64;
    static_assert(PER * NW <= TOPK_WG && 2 * PER * NW <= NC * CS, "one scan entry a thread");
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = i * TOPK_WG + lid;
        const bool valid = j < n;
        const uint64_t bg = __ballot(valid && key[i] > kth), be = __ballot(valid && key[i] == kth);
        if (lane == 0) {
            cg[i * NW + wv] = (uint32_t) __popcll(bg);
            ce[i * NW + wv] = (uint32_t) __popcll(be);
        }
    }
    __syncthreads();
    uint32_t total;
    const uint32_t mg = lid < PER * NW ? cg[lid] : 0u, me = lid < PER * NW ? ce[lid] : 0u;
    const uint32_t pg = wg_exclusive_scan(mg, wsum, total);
    const uint32_t pe = wg_exclusive_scan(me, wsum, total);
    if (lid < PER * NW) {
        cg[lid] = pg;
        ce[lid] = pe;
    }
    __syncthreads();
    const uint64_t below = ((uint64_t) 1 << lane) - 1;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = i * TOPK_WG + lid;
        const bool valid = j < n, gt = valid && key[i] > kth, eq = valid && key[i] == kth;
        const uint64_t bg = __ballot(gt), be = __ballot(eq);
        if (!(bg | be)) continue;                                  // (uniform: nothing of this wave's slice is taken)
        const uint32_t eq_before = ce[i * NW + wv] + (uint32_t) __popcll(be & below);
        const uint32_t at = cg[i * NW + wv] + (uint32_t) __popcll(bg & below) + std::min(eq_before, ties);
        if ((gt || (eq && eq_before < ties)) && at < (uint32_t) K) sel[r * K + at] = j;
    }
}

// A row's latent cells as a list (the prompt path that gathers them): row t of the pass sees, with a selection, the 4
// tokens of each of its sel_cnt[t] listed pools and then its incomplete pool's tokens 4 ((p + 1) / 4) .. p; without one
// (no counts, or a negative count) the cells 0 .. p. idx [T][NC] takes the first NC of them (0 past their end), n [T]
// their count, at most NC (kernels/llm/glm5next/glm.cpp:1023-1039)
__global__ __launch_bounds__(256) void glm_cells_kernel(const int32_t* __restrict__ sel, const int32_t* __restrict__ sel_cnt, int64_t T, int64_t K,
                                                        int64_t pos0, int32_t* __restrict__ idx, int32_t* __restrict__ n, int64_t NC) {
    const int64_t t = blockIdx.y;
    const int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (i >= NC) return;
    const int64_t pos = pos0 + t;
    const int64_t ns = sel_cnt ? sel_cnt[t] : -1;
    const int64_t tail0 = 4 * ((pos + 1) / 4);
    const int64_t cnt = ns < 0 ? pos + 1 : 4 * ns + (pos + 1 - tail0);
    int64_t c = 0;
    if (i < cnt) c = ns < 0 ? i : i < 4 * ns ? 4 * (int64_t) sel[t * K + i / 4] + i % 4 : tail0 + (i - 4 * ns);
    idx[t * NC + i] = (int32_t) c;
    if (i == 0) n[t] = (int32_t) std::min(cnt, NC);
}

// Row softmax of scores S [R H rows of NC]: row r's heads over its first n[r] cells, scaled; the rest of the row 0
// (kernels/llm/glm5next/glm.cpp:1041-1060). A work-group a row. VEC: 16-byte accesses (rows of a multiple of 4 cells at
// 16-byte aligned addresses), else one cell an access. Rows of up to 256 PER accesses stay in registers between the
// maximum, the sum and the division - one read and one write of the row, up to 32768 cells: the long rows of a prompt's
// chain are this kernel's everyday case - longer ones are read three times (PER = 0)
template <int PER, bool VEC>
__global__ __launch_bounds__(256) void glm_softmax_masked_kernel(float* __restrict__ S, int64_t H, int64_t NC, const int32_t* __restrict__ n, float scale) {
    constexpr int W = VEC ? 4 : 1;
    typedef float fw __attribute__((ext_vector_type(W)));
    __shared__ float red[8];
    const int64_t rh = blockIdx.x, r = rh / H;
    float* row = S + rh * NC;
    const int64_t m = std::min<int64_t>(std::max<int32_t>(n[r], 0), NC);
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    // access j of this thread: cells i0 .. i0 + W - 1, i0 = (tid + 256 j) W
    auto load = [&](int64_t i0) {
        fw v;
        if constexpr (VEC) {
            v = i0 < m ? *reinterpret_cast<const fw*>(row + i0) : fw{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int e = 0; e < W; ++e) v[e] = i0 + e < m ? v[e] * scale : -INFINITY;
        } else {
            v[0] = i0 < m ? row[i0] * scale : -INFINITY;
        }
        return v;
    };
    fw x[PER > 0 ? PER : 1];
    float mx = -INFINITY;
    if constexpr (PER > 0) {
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            x[j] = load((int64_t) (tid + 256 * j) * W);
#pragma unroll
            for (int e = 0; e < W; ++e) mx = fmaxf(mx, x[j][e]);
        }
    } else {
        for (int64_t i0 = (int64_t) tid * W; i0 < m; i0 += 256 * W) {
            const fw v = load(i0);
#pragma unroll
            for (int e = 0; e < W; ++e) mx = fmaxf(mx, v[e]);
        }
    }
    mx = wave_max(mx);
    if (lane == 0) red[wv] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float sum = 0.0f;
    if constexpr (PER > 0) {
#pragma unroll
        for (int j = 0; j < PER; ++j)
#pragma unroll
            for (int e = 0; e < W; ++e) {
                x[j][e] = x[j][e] == -INFINITY ? 0.0f : expf(x[j][e] - mx);
                sum += x[j][e];
            }
    } else {
        for (int64_t i0 = (int64_t) tid * W; i0 < m; i0 += 256 * W) {
            const fw v = load(i0);
#pragma unroll
            for (int e = 0; e < W; ++e) sum += v[e] == -INFINITY ? 0.0f : expf(v[e] - mx);
        }
    }
    sum = wave_sum(sum);
    if (lane == 0) red[4 + wv] = sum;
    __syncthreads();
    sum = (red[4] + red[5]) + (red[6] + red[7]);
    auto store = [&](int64_t i0, fw v) {
        if (i0 >= NC) return;
#pragma unroll
        for (int e = 0; e < W; ++e) v[e] = i0 + e < m ? v[e] / sum : 0.0f;
        if constexpr (VEC) *reinterpret_cast<fw*>(row + i0) = v;
        else row[i0] = v[0];
    };
    if constexpr (PER > 0) {
#pragma unroll
        for (int j = 0; j < PER; ++j) store((int64_t) (tid + 256 * j) * W, x[j]);
    } else {
        for (int64_t i0 = (int64_t) tid * W; i0 < NC; i0 += 256 * W) {
            fw v = load(i0);
#pragma unroll
            for (int e = 0; e < W; ++e) v[e] = v[e] == -INFINITY ? 0.0f : expf(v[e] - mx);
            store(i0, v);
        }
    }
}

}  // namespace

extern "C" {

int ns_idx_pool(ns_gpu* g, float* ring, const float* ik, const float* ig, const float* ape, float* pooled, int64_t pos0, int64_t T, int64_t D) {
    NS_TRY
    if (T <= 0 || D <= 0) return 0;
    if (pos0 < 0) return ns_fail("ns_idx_pool: a position");
    if (!g || !ring || !ik || !ig || !ape || !pooled) return ns_fail("ns_idx_pool: a null buffer");
    NS_HIP(hipSetDevice(g->dev));
    const int64_t j_lo = pos0 / 4, j_hi = (pos0 + T) / 4;
    if (j_hi > j_lo) {
        glm_idx_pool_kernel<<<(unsigned) (((j_hi - j_lo) * D + 255) / 256), 256, 0, g->q>>>(ring, ik, ig, ape, pooled, pos0, j_lo, j_hi - j_lo, D);
        NS_LAUNCHED("idx_pool");
    }
    const int64_t first = std::max<int64_t>(pos0, pos0 + T - 8);
    glm_idx_ring_kernel<<<(unsigned) (((pos0 + T - first) * D + 255) / 256), 256, 0, g->q>>>(ring, ik, ig, pos0, first, pos0 + T - first, D);
    NS_LAUNCHED("idx_pool ring");
    return 0;
    NS_CATCH
}

int ns_idx_score(ns_gpu* g, const float* S, const float* w, float* score, int64_t T, int64_t H, int64_t j0, int64_t n, int64_t ld, int64_t pos0) {
    NS_TRY
    if (T <= 0 || n <= 0) return 0;
    if (H < 0 || j0 < 0 || ld < j0 + n || pos0 < 0) return ns_fail("ns_idx_score: heads, a pool range inside a score row, a position");
    if (!g || !S || !w || !score) return ns_fail("ns_idx_score: a null buffer");
    NS_HIP(hipSetDevice(g->dev));
    glm_idx_score_kernel<<<(unsigned) ((T * n + 255) / 256), 256, 0, g->q>>>(S, w, score, T, H, j0, n, ld, pos0);
    NS_LAUNCHED("idx_score");
    return 0;
    NS_CATCH
}

int ns_topk(ns_gpu* g, const float* score, int32_t* sel, int64_t T, int64_t n, int64_t ld, int64_t K) {
    NS_TRY
    if (T <= 0 || K <= 0) return 0;
    // (fewer scores than K: the reference's select then takes all n, in position order, and leaves the list's rest as it was)
    if (n < 0 || ld < n || n > (int64_t) 1 << 30 || K > (int64_t) 1 << 30) return ns_fail("ns_topk: score rows at least n apart");
    if (!g || !score || !sel) return ns_fail("ns_topk: a null buffer");
    NS_HIP(hipSetDevice(g->dev));
    if (n <= 8 * TOPK_WG) glm_topk_reg_kernel<8><<<(unsigned) T, TOPK_WG, 0, g->q>>>(score, sel, (int) n, ld, (int) K);
    else if (n <= 32 * TOPK_WG) glm_topk_reg_kernel<32><<<(unsigned) T, TOPK_WG, 0, g->q>>>(score, sel, (int) n, ld, (int) K);
    else if (n <= 64 * TOPK_WG) glm_topk_reg_kernel<64><<<(unsigned) T, TOPK_WG, 0, g->q>>>(score, sel, (int) n, ld, (int) K);
    else glm_topk_kernel<<<(unsigned) T, TOPK_WG, 0, g->q>>>(score, sel, n, ld, K);
    NS_LAUNCHED("topk");
    return 0;
    NS_CATCH
}

int ns_mla_cells(ns_gpu* g, const int32_t* sel, const int32_t* sel_cnt, int64_t T, int64_t K, int64_t pos0, int32_t* idx, int32_t* n, int64_t NC) {
    NS_TRY
    if (T <= 0 || NC <= 0) return 0;
    if (sel_cnt && !sel) return ns_fail("ns_mla_cells: counts, but no lists");
    if (!g || !idx || !n) return ns_fail("ns_mla_cells: a null buffer");
    if (pos0 < 0 || K < 0 || pos0 + T > (int64_t) 1 << 31 || T > 65535) return ns_fail("ns_mla_cells: positions below 2^31, at most 65535 rows");
    NS_HIP(hipSetDevice(g->dev));
    glm_cells_kernel<<<dim3((unsigned) ((NC + 255) / 256), (unsigned) T), 256, 0, g->q>>>(sel, sel_cnt, T, K, pos0, idx, n, NC);
    NS_LAUNCHED("mla_cells");
    return 0;
    NS_CATCH
}

int ns_softmax_masked(ns_gpu* g, float* S, int64_t R, int64_t H, int64_t NC, const int32_t* n, float scale) {
    NS_TRY
    if (R <= 0 || H <= 0 || NC <= 0) return 0;
    if (!g || !S || !n) return ns_fail("ns_softmax_masked: a null buffer");
    if (R * H >= (int64_t) 1 << 31) return ns_fail("ns_softmax_masked: too many rows");
    NS_HIP(hipSetDevice(g->dev));
    const unsigned rows = (unsigned) (R * H);
    if (NC % 4 == 0 && (uintptr_t) S % 16 == 0) {
        if (NC <= 1024) glm_softmax_masked_kernel<1, true><<<rows, 256, 0, g->q>>>(S, H, NC, n, scale);
        else if (NC <= 4096) glm_softmax_masked_kernel<4, true><<<rows, 256, 0, g->q>>>(S, H, NC, n, scale);
        else if (NC <= 16384) glm_softmax_masked_kernel<16, true><<<rows, 256, 0, g->q>>>(S, H, NC, n, scale);
        else if (NC <= 32768) glm_softmax_masked_kernel<32, true><<<rows, 256, 0, g->q>>>(S, H, NC, n, scale);
        else glm_softmax_masked_kernel<0, true><<<rows, 256, 0, g->q>>>(S, H, NC, n, scale);
    } else {
        if (NC <= 256 * 4) glm_softmax_masked_kernel<4, false><<<rows, 256, 0, g->q>>>(S, H, NC, n, scale);
        else if (NC <= 256 * 16) glm_softmax_masked_kernel<16, false><<<rows, 256, 0, g->q>>>(S, H, NC, n, scale);
        else glm_softmax_masked_kernel<0, false><<<rows, 256, 0, g->q>>>(S, H, NC, n, scale);
    }
    NS_LAUNCHED("softmax_masked");
    return 0;
    NS_CATCH
}

int ns_llm_minimaxm3_idx_scores(ns_gpu* g, const float* iq, const uint16_t* ik, float* bs, int64_t T, int64_t G, int64_t nblk, int64_t pos0, int64_t local) {
    NS_TRY
    if (T <= 0 || G <= 0 || nblk <= 0) return 0;
    if (!iq || !ik || !bs) return ns_fail("ns_llm_minimaxm3_idx_scores: a null buffer");
    if ((uintptr_t) ik % 16) return ns_fail("ns_llm_minimaxm3_idx_scores: key rows 16-byte aligned");
    if (T * G * nblk > (int64_t) 1 << 31) return ns_fail("ns_llm_minimaxm3_idx_scores: too many blocks");
    NS_HIP(hipSetDevice(g->dev));
    // slices of whole 16-query stages, enough of them for ~4096 work-groups (16 a CU)
    const int64_t TG = T * G, stages = (TG + QCH - 1) / QCH;
    const int64_t slices = std::max<int64_t>(1, std::min<int64_t>({stages, (4096 + nblk - 1) / nblk, 65535}));
    const int64_t qper = (stages + slices - 1) / slices * QCH;
    idx_scores_kernel<<<dim3((unsigned) nblk, (unsigned) ((TG + qper - 1) / qper)), BLK, 0, g->q>>>(iq, ik, bs, TG, G, nblk, pos0, local, qper);
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
