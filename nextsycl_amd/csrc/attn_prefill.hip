// attn_prefill.hip: causal GQA flash attention of a prompt pass's rows against the KV cache (half or bfloat16 rows,
// D = 128) for gfx950.
//
// Bound: MFMA. 4 D flops a visible (row, key) pair against 2 x 2 D bytes a key shared by every row that sees it:
// thousands of flops a byte at prompt lengths.
//
// Work split: one work-group per (row block, query head). A work-group of 4 waves owns ROWS = 128 consecutive query rows
// of one query head (a wave 32 of them: two 16-row MFMA tiles) and streams the keys its rows see in 64-key tiles,
// heaviest row blocks first (the last block sees the most keys). The G query heads of a key head on one row block are
// neighbours in the logical order and, through the XCD-aware mapping of work-group ids, share one L2. A tile's K and V
// rows are fetched by all 256 threads (16-byte chunks): global -> registers two tiles ahead -> LDS one tile ahead, two
// register sets, two LDS buffers, one barrier a tile.
//
// A wave's tile step, in the transposed orientation (a lane owns one query row of each row tile, so the row maximum,
// the rescale and the normalisation never leave the lane):
//   S^T[key][row] = K Q^T        K from LDS as the A operand (ds_read_b128, rows padded to 272 bytes), Q^T in registers
//   base-2 online softmax in float32 (scale folded into the exponent's fma; the accumulators rescaled only when a
//   row's maximum moved); only 32-key halves crossing a row's causal or window edge are masked
//   P^T -> 16 bit = the B operand of the second product as it stands
//   O^T[d][row]  += V^T P^T      V^T from LDS through ds_read_b64_tr_b16 (rows padded to 288 bytes)
//
// Reference behaviour kept: kernels/llm/museglimmer/silo/attn.cpp:56-267 and kernels/llm/qwen35/silo/attn.cpp:105-313
// (prompt form: causal from p0, window, ring slots, 16-bit operands with float32 softmax and accumulation, rows past T
// not written, no scratch).
#include "ns_internal.hpp"
#include "ns_attn.h"
#include "attn_common.hpp"
#include "kv_formats.hpp"

#include <algorithm>
#include <cmath>
#include <type_traits>

namespace {

constexpr int PW = 4, ROWS = 128, KT_TILE = 64;

struct PrefillParams {
    const void* q;
    int qt;
    int64_t qs;
    const uint8_t* kc;
    const uint8_t* vc;
    int64_t head_stride, row_stride, cap;
    int wrap;
    int T, Hq, G;
    int64_t p0, win;
    float sl2;
    void* out;
};

// one thread's share of a 64-key tile on its way from global memory to LDS: 4 chunks of K, 4 of V
typedef uint32_t u4v __attribute__((ext_vector_type(4)));
struct Staged {
    u4v k[4], v[4];
};

template <int D, bool BF>
__global__ __launch_bounds__(PW * 64, 2) void attn_prefill_kernel(const PrefillParams p) {
    static_assert(D == 128, "head size 128");
    constexpr int KB = D / 32, DT = D / 16;
    constexpr int KS = D * 2 + 16, VS = D * 2 + 32;             // bytes a staged key row / value row
    constexpr int KBUF = KT_TILE * KS, VBUF = KT_TILE * VS;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * (KBUF + VBUF)];

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 15, g4 = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    // ---- which (row block, head) this work-group owns. Consecutive work-group ids go round the 8 XCDs (each with its
    // own L2): undo that, so that neighbours in the logical order - the G query heads of one key head on one row block,
    // which stream the same K / V tiles - share an L2. Logical order: heaviest row blocks first.
    const int nwg = gridDim.x, pid = blockIdx.x;
    const int xq = nwg / 8, xr = nwg % 8, xcd = pid % 8, xi = pid / 8;
    const int logical = (xcd < xr ? xcd * (xq + 1) : xr * (xq + 1) + (xcd - xr) * xq) + xi;
    const int nblk = (p.T + ROWS - 1) / ROWS;
    const int hq = logical % p.Hq;                               // heads fastest: hq / G is the key head
    const int blk = nblk - 1 - logical / p.Hq;
    const int hk = hq / p.G;
    const int r0 = blk * ROWS;
    const int rl = std::min(r0 + ROWS, p.T) - 1;                  // the block's last row
    const int64_t kend = p.p0 + rl + 1;                           // keys [kbeg, kend) cover every row of the block
    const int64_t kbeg = p.win > 0 ? std::max<int64_t>(0, p.p0 + r0 + 1 - p.win) : 0;

    // ---- this lane's two rows: positions, key ranges, Q^T operands
    int64_t lo_r[2], hi_r[2];
    s8v qreg[2][KB];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
        const int row = r0 + w * 32 + rt * 16 + n;
        const bool live = row < p.T;
        const int rr = live ? row : p.T - 1;
        const int64_t pos = p.p0 + rr;
        lo_r[rt] = live ? (p.win > 0 ? std::max<int64_t>(0, pos + 1 - p.win) : 0) : 1;
        hi_r[rt] = live ? pos : 0;
        const int64_t qoff = (int64_t) rr * p.qs + (int64_t) hq * D + g4 * 8;
        if (p.qt == 0) {
            float4 raw[KB][2];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                raw[kb][0] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.q) + qoff + kb * 32);
                raw[kb][1] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.q) + qoff + kb * 32 + 4);
            }
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                const float f[8] = {raw[kb][0].x, raw[kb][0].y, raw[kb][0].z, raw[kb][0].w, raw[kb][1].x, raw[kb][1].y, raw[kb][1].z, raw[kb][1].w};
#pragma unroll
                for (int i = 0; i < 8; ++i) qreg[rt][kb][i] = to16<BF>(f[i]);
            }
        } else {
            uint4 raw[KB];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) raw[kb] = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.q) + qoff + kb * 32);
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                const uint32_t ww[4] = {raw[kb].x, raw[kb].y, raw[kb].z, raw[kb].w};
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint16_t b16 = (uint16_t) (ww[i >> 1] >> (16 * (i & 1)));
                    qreg[rt][kb][i] = (p.qt == 2) == BF ? (short) b16 : to16<BF>(p.qt == 1 ? f16_to_f32(b16) : bf16_to_f32(b16));
                }
            }
        }
    }
    // the wave's own key range: its first row's first key to its last row's last (32-key halves outside are skipped)
    const int wrow0 = r0 + w * 32, wrow1 = std::min(wrow0 + 31, p.T - 1);
    const int64_t w_end = wrow0 < p.T ? p.p0 + wrow1 + 1 : 0;
    const int64_t w_beg = p.win > 0 ? std::max<int64_t>(0, p.p0 + wrow0 + 1 - p.win) : 0;
    // keys every row of the wave sees without a mask: [w_full_beg, w_full_end)
    const int64_t w_full_end = p.p0 + wrow0 + 1;
    const int64_t w_full_beg = p.win > 0 ? std::max<int64_t>(0, p.p0 + wrow1 + 1 - p.win) : 0;

    // running maximum in raw score units (the scale x log2(e) is folded into the exponent's fma), running sum of this
    // lane's own weights
    const float margin = 8.0f / p.sl2;
    float m_r[2] = {-INFINITY, -INFINITY}, l_r[2] = {0.0f, 0.0f};
    f4v o[2][DT];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[rt][dt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};

    const uint8_t* kbase = p.kc + (int64_t) hk * p.head_stride;
    const uint8_t* vbase = p.vc + (int64_t) hk * p.head_stride;
    const int64_t t0 = kbeg / KT_TILE, t1 = (kend + KT_TILE - 1) / KT_TILE;
    const int nt = (int) (t1 - t0);

    // a thread's chunks of a tile: chunk c = tid + 256 i -> key c / 16, 16-byte piece c % 16. Keys outside the block's
    // [kbeg, kend) are clamped into it (a valid row, masked; a tile past the last is fetched as the last row over and
    // over and never read). A wrapped ring's slot is position % cap: the first key's once, then offsets from it with at
    // most two wraps (a pass's keys span less than two rings)
    const int64_t kbeg_slot = p.wrap ? kbeg % p.cap : kbeg;
    const int kspan = (int) (kend - kbeg) - 1;
    const int key0 = tid >> 4;                                    // chunk i of this thread: key key0 + 16 i, piece tid & 15
    const uint8_t* kpiece = kbase + (tid & 15) * 16;
    const uint8_t* vpiece = vbase + (tid & 15) * 16;
    auto fetch = [&](Staged& st, int64_t ti) {
        const int rel0 = (int) (ti * KT_TILE - kbeg) + key0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int rel = std::min(std::max(rel0 + 16 * i, 0), kspan);
            int64_t slot = kbeg_slot + rel;
            if (p.wrap) {
                slot = slot >= p.cap ? slot - p.cap : slot;
                slot = slot >= p.cap ? slot - p.cap : slot;
            }
            const int64_t off = slot * p.row_stride;
            st.k[i] = *reinterpret_cast<const u4v*>(kpiece + off);
            st.v[i] = *reinterpret_cast<const u4v*>(vpiece + off);
        }
    };
    auto stash = [&](const Staged& st, int buf) {
        uint8_t* kb_ = lds + buf * (KBUF + VBUF);
        uint8_t* vb_ = kb_ + KBUF;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + PW * 64 * i, key = c >> 4, piece = c & 15;
            *reinterpret_cast<u4v*>(kb_ + key * KS + piece * 16) = st.k[i];
            *reinterpret_cast<u4v*>(vb_ + key * VS + piece * 16) = st.v[i];
        }
    };

    // one 32-key half of a staged tile against this wave's 32 rows. LDS is addressed with 32-bit offsets from the
    // array's start (kl, vl: byte offsets); the mask is applied under a wave-uniform branch, so halves no row edge
    // crosses - nearly all of them - pay for no comparison
    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    lds_u8* const L = (lds_u8*) lds;
    const uint32_t k_rd = (uint32_t) (n * KS + g4 * 16);                          // + kt2 * 16 * KS + kb * 64
    const uint32_t v_rd = (uint32_t) ((g4 * 4 + (n >> 2)) * VS + (n & 3) * 8);    // + dt * 32 (+ 16 * VS)
    auto half = [&](uint32_t kl, uint32_t vl, int64_t j0, bool masked) {
        // ---- S^T = K Q^T
        f4v s[2][2];
#pragma unroll
        for (int kt2 = 0; kt2 < 2; ++kt2) {
            s8v ka[KB];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
                ka[kb] = *reinterpret_cast<const __attribute__((address_space(3))) s8v*>(L + kl + k_rd + kt2 * 16 * KS + kb * 64);
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                f4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) acc = mfma16<BF>(ka[kb], qreg[rt][kb], acc);
                s[rt][kt2] = acc;
            }
        }
        // ---- softmax
        s8v pb[2];
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            float x[8];
#pragma unroll
            for (int kt2 = 0; kt2 < 2; ++kt2)
#pragma unroll
                for (int i = 0; i < 4; ++i) x[kt2 * 4 + i] = s[rt][kt2][i];
            if (masked) {
                // keys lo .. hi of this half (relative, clamped into 0 .. 32 / -1 .. 31) are the row's: one unsigned
                // compare a key
                const int lo = (int) std::min<int64_t>(std::max<int64_t>(lo_r[rt] - j0, 0), 32);
                const int hi = (int) std::min<int64_t>(std::max<int64_t>(hi_r[rt] - j0, -1), 31);
                const unsigned span = (unsigned) (hi - lo);          // hi < lo: no key, and span wraps to huge...
                const bool none = hi < lo;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int j = (e >> 2) * 16 + g4 * 4 + (e & 3);
                    x[e] = (!none && (unsigned) (j - lo) <= span) ? x[e] : -INFINITY;
                }
            }
            // The running maximum m_r is moved - and the accumulators rescaled - only when some score of the wave
            // outgrows it by more than 2^8 after scaling; otherwise the weights are taken against the maximum as it
            // stands (they may then exceed 1, by at most 2^8: harmless in float32 sums and 16-bit operands, and the
            // final division by l makes the result the same function of the inputs). The common path therefore has
            // no cross-lane step at all: a lane checks its own 8 scores.
            const float mxl = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
            if (__any(mxl > m_r[rt] + margin)) {
                const float mn = fmaxf(m_r[rt], rows_max(mxl));
                const float c = mn == -INFINITY ? 1.0f : fast_exp2((m_r[rt] - mn) * p.sl2);
                l_r[rt] *= c;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) o[rt][dt] *= c;
                m_r[rt] = mn;
            }
            const float nb = m_r[rt] == -INFINITY ? 0.0f : -m_r[rt] * p.sl2;
            float sum = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float pv = fast_exp2(__builtin_fmaf(x[e], p.sl2, nb));   // x = -inf -> 0
                sum += pv;
                pb[rt][e] = to16<BF>(pv);
            }
            l_r[rt] += sum;                                        // this lane's keys only: reduced over the row at the end
        }
        // ---- O^T += V^T P^T
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const s4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*) (L + vl + v_rd + dt * 32));
            const s4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*) (L + vl + v_rd + dt * 32 + 16 * VS));
            const s8v va = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) o[rt][dt] = mfma16<BF>(va, pb[rt], o[rt][dt]);
        }
    };
    auto compute = [&](int buf, int64_t ti) {
        const uint32_t kl = (uint32_t) (buf * (KBUF + VBUF)), vl = kl + KBUF;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int64_t j0 = ti * KT_TILE + h * 32;
            if (j0 < w_end && j0 + 32 > w_beg) {
                half(kl + h * 32 * KS, vl + h * 32 * VS, j0, !(j0 >= w_full_beg && j0 + 32 <= w_full_end));
            }
        }
    };

    // ---- the pipeline: tile k computed from LDS buffer k & 1 while tile k + 1 sits in registers (written to the other
    // buffer at the iteration's end) and tile k + 2 is on its way from global memory. Fetches and stashes past the last
    // tile are harmless repeats, so that no register array is conditionally defined
    if (nt > 0) {
        Staged sa, sb;
        fetch(sa, t0);
        fetch(sb, t0 + 1);
        stash(sa, 0);
        __syncthreads();
        for (int k = 0; k < nt; k += 2) {
            fetch(sa, t0 + k + 2);
            compute(0, t0 + k);
            stash(sb, 1);
            __syncthreads();
            if (k + 1 >= nt) break;
            fetch(sb, t0 + k + 3);
            compute(1, t0 + k + 1);
            stash(sa, 0);
            __syncthreads();
        }
    }

    // ---- out = O / l; a lane holds dims 16 dt + 4 g4 .. + 3 of its rows
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
        const int row = r0 + w * 32 + rt * 16 + n;
        const float lsum = rows_sum(l_r[rt]);                 // every lane takes part, dead rows too
        if (row >= p.T) continue;
        const float inv = lsum > 0.0f ? 1.0f / lsum : 0.0f;
        const int64_t at = ((int64_t) row * p.Hq + hq) * D + g4 * 4;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const f4v v = o[rt][dt] * inv;
            if (p.qt == 0) {
                *reinterpret_cast<f4v*>(reinterpret_cast<float*>(p.out) + at + dt * 16) = v;
            } else {
                ushort4 h;
                if (p.qt == 1) h = make_ushort4(f32_to_f16(v[0]), f32_to_f16(v[1]), f32_to_f16(v[2]), f32_to_f16(v[3]));
                else h = make_ushort4(f32_to_bf16(v[0]), f32_to_bf16(v[1]), f32_to_bf16(v[2]), f32_to_bf16(v[3]));
                *reinterpret_cast<ushort4*>(reinterpret_cast<uint16_t*>(p.out) + at + dt * 16) = h;
            }
        }
    }
}

}  // namespace

int ns_attn_prompt_any(ns_gpu* g, const char* who, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T,
                       int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, float scale, void* out) {
    NS_TRY
    const std::string w(who);
    if (T <= 0) return 0;
    if (D != 128) return ns_fail(w + ": heads of 128");
    if (Hkv <= 0 || Hq <= 0 || Hq % Hkv) return ns_fail(w + ": query heads a multiple of the key heads");
    if (kt != 0 && kt != 3) return ns_fail(w + ": a cache form 0 (half) or 3 (bfloat16)");
    if (qt < 0 || qt > 2) return ns_fail(w + ": rows of type 0 (float32), 1 (half) or 2 (bfloat16)");
    if (p0 < 0 || cap <= 0) return ns_fail(w + ": a position and a capacity");
    const int64_t need = pm ? p0 + T : (win > 0 ? std::min(p0 + T, win + T - 1) : p0 + T);
    if (need > cap) return ns_fail(w + (win > 0 ? ": the cache's ring is shorter than the window and the pass" : ": past the cache's capacity"));
    if (!q || !kc || !vc || !out) return ns_fail(w + ": a null buffer");
    if ((uintptr_t) q % 16 || qs % (qt == 0 ? 4 : 8) || (uintptr_t) out % 16) return ns_fail(w + ": query and output rows 16-byte aligned");
    if (((uintptr_t) kc | (uintptr_t) vc) % 16) return ns_fail(w + ": caches 16-byte aligned");
    if (T > (int64_t) 1 << 30 || ((T + ROWS - 1) / ROWS) * Hq > (int64_t) 1 << 30) return ns_fail(w + ": too many rows or heads");
    NS_HIP(hipSetDevice(g->dev));
    const int64_t rb = 2 * D;
    PrefillParams p{};
    p.q = q;
    p.qt = qt;
    p.qs = qs;
    p.kc = (const uint8_t*) kc;
    p.vc = (const uint8_t*) vc;
    p.head_stride = pm ? rb : cap * rb;
    p.row_stride = pm ? Hkv * rb : rb;
    p.cap = cap;
    p.wrap = !pm && p0 + T > cap;
    p.T = (int) T;
    p.Hq = (int) Hq;
    p.G = (int) (Hq / Hkv);
    p.p0 = p0;
    p.win = win;
    p.sl2 = (scale > 0.0f ? scale : 1.0f / sqrtf((float) D)) * 1.4426950408889634f;
    p.out = out;
    dim3 grid((unsigned) (((T + ROWS - 1) / ROWS) * Hq));
    if (ns_profile_mark(g, 0)) return -1;
    if (kt == 3) attn_prefill_kernel<128, true><<<grid, PW * 64, 0, g->q>>>(p);
    else attn_prefill_kernel<128, false><<<grid, PW * 64, 0, g->q>>>(p);
    NS_LAUNCHED("attn_prefill");
    return ns_profile_mark(g, 1);
    NS_CATCH
}

extern "C" {

int ns_attn_prompt_t(ns_gpu* g, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq,
                     int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, float scale, void* out) {
    return ns_attn_prompt_any(g, "ns_attn_prompt_t", qt, kt, pm, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, win, scale, out);
}

}  // extern "C"
