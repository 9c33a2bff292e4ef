// pre_attn.hip: what runs in front of attention on every token - q / k RMS norm, rotary positions, the KV store - for
// gfx950: the reference's separate entry points and one fused launch (norm + rotate + store, k never written as
// float32). Bound: HBM - a few KB a token at a decode step (the point of the fused form is two launches fewer a layer),
// (Hq + 2 Hkv) D 4 bytes read and about half that written a row in a prompt pass.
//
// One wave a (row, head) - two or four rows of a head where a head row is 128 or 64 features, so no lane idles; a lane
// four consecutive features (D up to 256; more: a lane two groups of four). In a prompt pass a wave walks several heads
// of its rows on one evaluation of the rotation, the next head's loads in flight while it works on this one. Every load
// of a head precedes its stores, so source and destination may be the same rows. The arithmetic of an output feature
// is the same whatever entry point asks for it, and the quantized rows are kv_pack.hpp's: the fused launch gives bit
// for bit what the separate calls give. Compiled with -ffp-contract=off (the packers).
//
// Reference behaviour kept: kernels/llm/qwen35/q35.cpp:220-279,350-386 (rotate-half over the first n_rot, angle
// pos * theta^(-2 k / n_rot); interleaved position sections), kernels/llm/museglimmer/mg.cpp:157-190 (adjacent pairs or
// halves over all D), kernels/llm/minimaxm3/mm3.cpp:18-35 and silo/moe.cpp:460-501 (angle by repeated multiplication,
// norm as 1 / sqrt).
#include "ns_internal.hpp"
#include "ns_pre.h"
#include "kv_formats.hpp"
#include "kv_pack.hpp"
#include "attn_common.hpp"
#include "attn_host.hpp"

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdlib>
#include <type_traits>

namespace {

enum { ROPE_NONE = 0, ROPE_Q35 = 1, ROPE_MG_PAIRS = 2, ROPE_MG_HALVES = 3, ROPE_MM3 = 4 };
// where a group's rows go: float32 / half / bfloat16 rows [t * ds + h * D], or cache rows of form kt
enum { DST_F32 = 0, DST_F16 = 1, DST_BF16 = 2, DST_CACHE = 8 };

struct PreGroup {
    int heads;                 // heads of this group in a row t
    const float* src;
    int64_t ss, hs;            // floats between rows / heads of src
    const float* w;            // norm weight [D], or null: no norm
    int rope;                  // rotate this group
    void* dst;
    int64_t ds;                // elements between dst rows (plain destinations)
    int dt;                    // DST_*; DST_CACHE + kt for cache rows
    void* dst2;                // a second, half copy of the result (minimaxm3's in-place rows also stored as half), or null
    int64_t ds2;
};

struct PreParams {
    PreGroup gr[5];
    int ngr;
    int T, D;
    int mode, n_rot, inv_sqrt;        // inv_sqrt: 1 / sqrt(..) instead of rsqrt(..)
    float theta, ts, eps;
    int64_t p0;
    const int32_t* pos3;              // [T][3] positions, or null
    int s0, s1, s2;
    int64_t cap;
    int ring;
    int hpw;                          // heads of a row a wave walks (their rotation worked out once)
};

// the rotation of output feature i at row t: cosine and sine of its angle (on = false: the feature is not rotated). It
// depends on the row and the feature only - not on the head - so a wave that walks several heads of a row works it out
// once: powf, cosf and sinf are most of this kernel's arithmetic
struct Rot {
    float c, s;
    bool on;
};
__device__ __forceinline__ Rot rope_cs(const PreParams& p, int i, int t) {
    Rot r{1.0f, 0.0f, false};
    if (p.mode == ROPE_NONE) return r;
    const int D = p.D;
    if (p.mode == ROPE_Q35) {
        if (i >= p.n_rot) return r;
        const int hr = p.n_rot / 2, k = i < hr ? i : i - hr;
        float pos = (float) (p.p0 + t);
        if (p.pos3) {
            const int sect = p.s0 + p.s1 + p.s2, sec = k % sect;
            const int c = (sec % 3 == 1 && sec < 3 * p.s1) ? 1 : (sec % 3 == 2 && sec < 3 * p.s2) ? 2 : 0;
            pos = (float) p.pos3[t * 3 + c];
        }
        const float a = pos * powf(p.theta, -2.0f * (float) k / (float) p.n_rot);
        float sn, cs;
        sincosf(a, &sn, &cs);          // (one argument reduction for both)
        return Rot{cs, sn, true};
    }
    if (p.mode == ROPE_MG_PAIRS || p.mode == ROPE_MG_HALVES) {
        const bool halves = p.mode == ROPE_MG_HALVES;
        const int pr = halves ? (i < D / 2 ? i : i - D / 2) : i / 2;
        const float a = (float) (p.p0 + t) * powf(p.theta, -2.0f * (float) pr / (float) D);
        float sn, cs;
        sincosf(a, &sn, &cs);          // (one argument reduction for both)
        return Rot{cs, sn, true};
    }
    // ROPE_MM3
    if (i >= p.n_rot) return r;
    const int hr = p.n_rot / 2, k = i % hr;
    float th = (float) (p.p0 + t);
    for (int j = 0; j < k; ++j) th *= p.ts;
    float sn, cs;
    sincosf(th, &sn, &cs);
    return Rot{cs, sn, true};
}

// output feature i of a head row: v(j) = x[j] * inv * w[j] (or x[j]), rotated as the mode says by r = rope_cs(p, i, t)
__device__ __forceinline__ float rope_feature(const PreParams& p, const float* x, const float* w, float inv, int i, bool rot, const Rot& r) {
    auto v = [&](int j) { return w ? x[j] * inv * w[j] : x[j]; };
    const float me = v(i);
    if (!rot || !r.on) return me;
    const int D = p.D;
    const float c = r.c, sn = r.s;
    if (p.mode == ROPE_Q35) {
        const int hr = p.n_rot / 2;
        const float other = v(i < hr ? i + hr : i - hr);
        return i < hr ? me * c - other * sn : me * c + other * sn;
    }
    if (p.mode == ROPE_MG_PAIRS || p.mode == ROPE_MG_HALVES) {
        const bool halves = p.mode == ROPE_MG_HALVES;
        const int pr = halves ? (i < D / 2 ? i : i - D / 2) : i / 2;
        const int i0 = halves ? pr : 2 * pr, i1 = halves ? pr + D / 2 : 2 * pr + 1;
        const float a0 = i == i0 ? me : v(i0), a1 = i == i1 ? me : v(i1);
        return i == i0 ? a0 * c - a1 * sn : a0 * sn + a1 * c;
    }
    // ROPE_MM3
    const int hr = p.n_rot / 2;
    const float them = v(i < hr ? i + hr : i - hr);
    return i < hr ? me * c - them * sn : them * sn + me * c;
}

// VEC: whole 4-feature groups pair up under the rotation (see below); MAXG: 4-feature groups a lane (1: D up to 256)
// DC: the head size when it is 128 or 256 - a head row then fills its lanes exactly (no lane idles, no feature past the row)
// and the reduction over a row's lanes has no branch - else 0: any size, read from the arguments.
// 4 waves a SIMD (128 registers) for the form that serves the engines' sizes: measured best - 76 against 82 us at 8192 rows x
// 56 heads with the allocation left alone (138 registers, 3 waves); the other forms keep at least 2
template <bool VEC, int MAXG, int DC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(VEC && MAXG == 1 ? 4 : 2, 4))) void pre_attn_kernel(const PreParams p) {
    const int lane = threadIdx.x & 63;
    const int D = DC ? DC : p.D;
    // (DC: every lane holds 4 features of a row; a row past the last loads the last row again and stores nothing - its sums
    // stay among its own lanes - so nothing has to be zeroed)
    constexpr bool EXACT = DC != 0;
    // a head row of 64 or 128 features takes 16 or 32 lanes: the wave then carries 4 or 2 consecutive rows t of the same
    // head at once (same group, same weights; the rotation is a lane's own anyway), and no lane idles
    const int lph = DC == 128 ? 32 : DC == 256 ? 64 : MAXG == 1 && D == 64 ? 16 : MAXG == 1 && D == 128 ? 32 : 64;
    const int rpw = 64 / lph, sub = lane / lph, li = lane - sub * lph;
    // the wave's index as a scalar: the row, the head and its group's descriptor then live in scalar registers
    const int64_t wid = (int64_t) blockIdx.x * 4 + __builtin_amdgcn_readfirstlane((int) (threadIdx.x >> 6));
    int per_t = 0;
#pragma unroll
    for (int gi = 0; gi < 5; ++gi) per_t += gi < p.ngr ? p.gr[gi].heads : 0;
    const int wpt = (per_t + p.hpw - 1) / p.hpw;           // waves a group of rows: each walks hpw of the rows' heads
    if (wid >= (int64_t) ((p.T + rpw - 1) / rpw) * wpt) return;   // whole waves leave: no shuffle below misses a lane
    const int t = (int) (wid / wpt) * rpw + sub;
    const bool row_live = t < p.T;                         // a lane past the last row loads zeros and stores nothing
    const int hfirst = (int) (wid % wpt) * p.hpw, hend = min(hfirst + p.hpw, per_t);
    // the rotation of this lane's features at this row: the same for every head. One copy of the angle code, looped (eight
    // unrolled copies cost the kernel half its waves in registers); the results go to registers by constant index
    float rc[MAXG * 4], rs[MAXG * 4];
    uint32_t onmask = 0;
#pragma unroll
    for (int q = 0; q < MAXG * 4; ++q) rc[q] = 1.0f, rs[q] = 0.0f;
    const int nfeat = MAXG == 1 || D <= 256 ? 4 : 8;
#pragma nounroll
    for (int e = 0; e < nfeat; ++e) {
        const int i = li * 4 + (e >> 2) * 256 + (e & 3);
        const Rot r = i < D && row_live ? rope_cs(p, i, t) : Rot{1.0f, 0.0f, false};
#pragma unroll
        for (int q = 0; q < MAXG * 4; ++q)
            if (q == e) rc[q] = r.c, rs[q] = r.s;
        onmask |= (r.on ? 1u : 0u) << e;
    }
    // the distance to a rotated feature's partner
    const int pdist = p.mode == ROPE_MG_HALVES ? D / 2 : p.n_rot / 2;
    // Every rotary form is y = me cos -/+ partner sin, minus for the first feature of a pair (a - b is a + (-b) bit for
    // bit, and the forms that write the sum the other way round add the same two products): the sign goes into the sine
    // once, and a feature is one multiply-add pair with no branch. (VEC only; the other instance keeps rope_feature.)
    float rss[MAXG * 4];
#pragma unroll
    for (int q = 0; q < MAXG * 4; ++q) {
        const int i = li * 4 + (q >> 2) * 256 + (q & 3);
        const bool first = p.mode == ROPE_MG_PAIRS ? (q & 1) == 0 : i < pdist;
        rss[q] = first ? -rs[q] : rs[q];
    }
    const bool d_pow2 = (D & (D - 1)) == 0;
    const float inv_d = 1.0f / (float) D;                  // exact for a power of two: s * inv_d is s / D bit for bit
    // The wave walks its heads group by group: a group's descriptor (scalar registers, read from the kernel-argument block
    // at a scalar index - indexing the by-value argument at run time would send it through private memory), the lane's row
    // bases in the group's source and destination, its weights and which of its features the group rotates are worked out
    // once a group; a head then costs two 64-bit additions an address, its loads, its arithmetic and its stores.
    // Every load is unconditional - a lane with nothing to do reads a valid address and drops the value - so the loads
    // of the next two heads are in flight while this head is worked on
    struct HeadIn {
        const float* x;
        float4 xo[MAXG], xp[MAXG];
    };
    const int tl = row_live ? t : p.T - 1;
    const PreGroup* groups = reinterpret_cast<const PreGroup*>((const char*) __builtin_amdgcn_kernarg_segment_ptr() + offsetof(PreParams, gr));
    int gfirst = 0;
    for (int gi = 0; gi < p.ngr; ++gi) {
    const PreGroup G = groups[gi];
    const int g0 = gfirst;
    gfirst += G.heads;
    const int ha = max(hfirst, g0) - g0, hb = min(hend, gfirst) - g0;     // this wave's heads of the group
    if (ha >= hb) continue;
    // ---- once a group: the lane's own features and their partners in the row, the weights of both
    const float* xrow = G.src + (int64_t) tl * G.ss;
    int io[MAXG], ipn[MAXG];
    bool rot_c[MAXG];
    float4 wo[MAXG], wp[MAXG];
#pragma unroll
    for (int c = 0; c < MAXG; ++c) {
        const int i0 = li * 4 + c * 256, i = i0 < D ? i0 : 0;
        rot_c[c] = G.rope != 0 && (onmask >> (c * 4) & 1) != 0;
        io[c] = i;
        ipn[c] = !rot_c[c] || p.mode == ROPE_MG_PAIRS ? i : i < pdist ? i + pdist : i - pdist;
        if constexpr (VEC) {
            const float* w = G.w ? G.w : xrow;
            wo[c] = *reinterpret_cast<const float4*>(w + io[c]);
            wp[c] = *reinterpret_cast<const float4*>(w + ipn[c]);
        }
    }
    auto fetch = [&](int h, HeadIn& in) __attribute__((always_inline)) {
        in.x = xrow + (int64_t) h * G.hs;
#pragma unroll
        for (int c = 0; c < MAXG; ++c) {
            in.xo[c] = *reinterpret_cast<const float4*>(in.x + io[c]);
            if constexpr (VEC) in.xp[c] = *reinterpret_cast<const float4*>(in.x + ipn[c]);
        }
    };
    // where the lane's results go: a plain row's element (t, h = 0, feature i), or the cache row of head 0 at the row's slot
    const int64_t slot = p.ring ? (p.p0 + t) % p.cap : p.p0 + t;
    const int64_t rb = G.dt >= DST_CACHE ? kv_row_bytes(G.dt - DST_CACHE, D) : 0;
    uint8_t* const crow0 = reinterpret_cast<uint8_t*>(G.dst) + slot * rb;
    const int64_t at0 = (int64_t) t * G.ds, at20 = (int64_t) t * G.ds2;
    // the group's heads, one copy of the loop a destination form and "has weights" (both are the group's, not a head's:
    // decided here, the loop holds no select or branch on them)
    auto walk = [&](auto dt_c, auto w_c) __attribute__((always_inline)) {
    constexpr int DTK = decltype(dt_c)::value;
    constexpr bool HASW = decltype(w_c)::value;
    constexpr int kt = DTK - DST_CACHE;
    // one head: its row's scale, its features, its stores
    auto head = [&](int h, const HeadIn& cur) __attribute__((always_inline)) {
    const float* x = cur.x;
    // ---- the row's scale
    float4 xo[MAXG];
#pragma unroll
    for (int c = 0; c < MAXG; ++c) xo[c] = EXACT || (li * 4 + c * 256 < D && row_live) ? cur.xo[c] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    float inv = 1.0f;
    if constexpr (HASW) {
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < MAXG; ++c) {
            s += xo[c].x * xo[c].x;
            s += xo[c].y * xo[c].y;
            s += xo[c].z * xo[c].z;
            s += xo[c].w * xo[c].w;
        }
        // over the head row's lanes, pairwise as an exclusive-or butterfly would (lanes past the row carry zeros)
        s = row16_sum(s);
        float a, b;
        if (lph > 16) {
            pair16(s, a, b);
            s = a + b;
        }
        if (lph > 32) {
            pair32(s, a, b);
            s = a + b;
        }
        const float ms = (d_pow2 ? s * inv_d : s / (float) D) + p.eps;
        inv = p.inv_sqrt ? 1.0f / sqrtf(ms) : rsqrtf(ms);
    }
    // ---- this lane's features. Where the partner of a rotated feature lies a whole number of 4-feature groups away
    // (or inside the lane's own group: adjacent pairs) the partners came in one 16-byte load as well; other widths
    // take the feature-by-feature form
    float y[MAXG][4];
    if constexpr (VEC) {
#pragma unroll
        for (int c = 0; c < MAXG; ++c) {
            const int i = li * 4 + c * 256;
            if (!EXACT && (i >= D || !row_live)) {
#pragma unroll
                for (int j = 0; j < 4; ++j) y[c][j] = 0.0f;
                continue;
            }
            const bool rotated = rot_c[c];
            const float4 xp4 = cur.xp[c], wo4 = wo[c], wp4 = wp[c];
            const float xv[4] = {xo[c].x, xo[c].y, xo[c].z, xo[c].w}, xq[4] = {xp4.x, xp4.y, xp4.z, xp4.w};
            const float wv[4] = {wo4.x, wo4.y, wo4.z, wo4.w}, wq[4] = {wp4.x, wp4.y, wp4.z, wp4.w};
            float me[4], pt[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                me[j] = HASW ? xv[j] * inv * wv[j] : xv[j];
                pt[j] = HASW ? xq[j] * inv * wq[j] : xq[j];
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float other = p.mode == ROPE_MG_PAIRS ? me[j ^ 1] : pt[j];
                const float r = me[j] * rc[c * 4 + j] + other * rss[c * 4 + j];
                y[c][j] = rotated ? r : me[j];
            }
        }
    } else {
#pragma unroll
        for (int c = 0; c < MAXG; ++c) {
            const int i = li * 4 + c * 256;
#pragma unroll
            for (int j = 0; j < 4; ++j) y[c][j] = i < D && row_live ? rope_feature(p, x, HASW ? G.w : nullptr, inv, i + j, G.rope != 0, Rot{rc[c * 4 + j], rs[c * 4 + j], (onmask >> (c * 4 + j) & 1) != 0}) : 0.0f;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");   // loads above, stores below (source may be destination)
#pragma unroll
    for (int c = 0; c < MAXG; ++c) {
        const int i = li * 4 + c * 256;
        if (c * 256 >= D) break;
        const bool live = i < D && row_live;
        if constexpr (DTK < DST_CACHE) {
            if (!live) continue;
            const int64_t at = at0 + (int64_t) h * D + i;
            if constexpr (DTK == DST_F32) {
                *reinterpret_cast<float4*>(reinterpret_cast<float*>(G.dst) + at) = make_float4(y[c][0], y[c][1], y[c][2], y[c][3]);
            } else {
                ushort4 o;
                if constexpr (DTK == DST_F16) o = make_ushort4(f32_to_f16(y[c][0]), f32_to_f16(y[c][1]), f32_to_f16(y[c][2]), f32_to_f16(y[c][3]));
                else o = make_ushort4(f32_to_bf16(y[c][0]), f32_to_bf16(y[c][1]), f32_to_bf16(y[c][2]), f32_to_bf16(y[c][3]));
                *reinterpret_cast<ushort4*>(reinterpret_cast<uint16_t*>(G.dst) + at) = o;
            }
            if (G.dst2) {
                const int64_t at2 = at20 + (int64_t) h * D + i;
                *reinterpret_cast<ushort4*>(reinterpret_cast<uint16_t*>(G.dst2) + at2) =
                    make_ushort4(f32_to_f16(y[c][0]), f32_to_f16(y[c][1]), f32_to_f16(y[c][2]), f32_to_f16(y[c][3]));
            }
        } else {
            uint8_t* row = crow0 + (int64_t) h * p.cap * rb;
            if constexpr (kt == 0 || kt == 3) {
                if (!live) continue;
                ushort4 o;
                if constexpr (kt == 0) o = make_ushort4(f32_to_f16(y[c][0]), f32_to_f16(y[c][1]), f32_to_f16(y[c][2]), f32_to_f16(y[c][3]));
                else o = make_ushort4(f32_to_bf16(y[c][0]), f32_to_bf16(y[c][1]), f32_to_bf16(y[c][2]), f32_to_bf16(y[c][3]));
                *reinterpret_cast<ushort4*>(row + 2 * i) = o;
            } else {
                // 8 lanes a block of 32: every lane takes part in the shuffles (dead lanes carry zeros, store nothing)
                const int b = i / 32, ln = li & 7;
                float d;
                if constexpr (kt == 1) {
                    const uint32_t wv = q8_0_pack4(y[c], d);
                    if (live) {
                        *reinterpret_cast<uint32_t*>(row + i) = wv;
                        if (ln == 0) *reinterpret_cast<uint16_t*>(row + D + 2 * b) = f32_to_f16(d);
                    }
                } else {
                    const uint32_t wv = q4_0_pack4(y[c], ln, d);
                    if (live && ln < 4) {
                        *reinterpret_cast<uint32_t*>(row + b * 16 + ln * 4) = wv;
                        if (ln == 0) *reinterpret_cast<uint16_t*>(row + D / 2 + 2 * b) = f32_to_f16(d);
                    }
                }
            }
        }
    }
    };
    // The group's heads, the loads two heads ahead of the arithmetic: three register sets taken in turn by name (a set
    // handed on by copy would wait for the newest load - the copy reads it - and nothing would be in flight under the
    // arithmetic). The last heads read the last again rather than branch
    HeadIn in0, in1, in2;
    fetch(ha, in0);
    fetch(ha + 1 < hb ? ha + 1 : ha, in1);
    for (int h = ha;;) {
        fetch(h + 2 < hb ? h + 2 : hb - 1, in2);
        head(h, in0);
        if (++h >= hb) break;
        fetch(h + 2 < hb ? h + 2 : hb - 1, in0);
        head(h, in1);
        if (++h >= hb) break;
        fetch(h + 2 < hb ? h + 2 : hb - 1, in1);
        head(h, in2);
        if (++h >= hb) break;
    }
    };
    auto walk_w = [&](auto w_c) __attribute__((always_inline)) {
        switch (G.dt) {
            case DST_F32: walk(std::integral_constant<int, DST_F32>{}, w_c); break;
            case DST_F16: walk(std::integral_constant<int, DST_F16>{}, w_c); break;
            case DST_BF16: walk(std::integral_constant<int, DST_BF16>{}, w_c); break;
            case DST_CACHE + 0: walk(std::integral_constant<int, DST_CACHE + 0>{}, w_c); break;
            case DST_CACHE + 1: walk(std::integral_constant<int, DST_CACHE + 1>{}, w_c); break;
            case DST_CACHE + 2: walk(std::integral_constant<int, DST_CACHE + 2>{}, w_c); break;
            default: walk(std::integral_constant<int, DST_CACHE + 3>{}, w_c); break;
        }
    };
    if (G.w) walk_w(std::true_type{});
    else walk_w(std::false_type{});
    }   // the wave's next group
}

int launch_pre(ns_gpu* g, const PreParams& p, const char* who) {
    NS_HIP(hipSetDevice(g->dev));
    int64_t per_t = 0;
    for (int i = 0; i < p.ngr; ++i) per_t += p.gr[i].heads;
    if (per_t <= 0 || p.T <= 0) return 0;
    // a wave a (row group, head) while that leaves the chip short of waves (a decode step); a prompt's rows have waves to
    // spare, and each then walks several heads of its rows on one evaluation of the rotation (most of a wave's
    // arithmetic, as much as some 16 heads). The waves' arithmetic is what a pass of some hundred rows and more waits for, so
    // fewer, longer waves win until too few are left to keep memory busy: about 2048 waves a launch measured best (512 rows
    // x 56 heads: 1 / 4 / 7 / 14 / 28 heads a wave 27.2 / 11.6 / 9.9 / 11.2 / 14.7 us; 2048 rows: 7 / 14 / 28 heads 23.3 /
    // 19.9 / 19.3; 8192 rows: 14 / 28 / 56 heads 76.7 / 73.7 / 74.7), the heads of a row group shared evenly among its waves
    PreParams q = p;
    const int64_t rpw = p.D == 64 ? 4 : p.D == 128 ? 2 : 1, tg = (p.T + rpw - 1) / rpw;
    q.hpw = (int) std::max<int64_t>(1, std::min<int64_t>(per_t, (tg * per_t + 2047) / 2048));
    q.hpw = (int) ((per_t + (per_t + q.hpw - 1) / q.hpw - 1) / ((per_t + q.hpw - 1) / q.hpw));
    if (const int64_t forced = ns_tune_get(NS_TUNE_PRE_HPW)) q.hpw = (int) std::max<int64_t>(1, std::min<int64_t>(per_t, forced));   // sweeps
    const int64_t waves = tg * ((per_t + q.hpw - 1) / q.hpw);
    if ((waves + 3) / 4 > (int64_t) 1 << 31) return ns_fail(std::string(who) + ": too many rows");
    // whole 4-feature groups pair up: no rotation, adjacent pairs, or partners a multiple of 4 features away
    const bool vec = p.mode == ROPE_NONE || p.mode == ROPE_MG_PAIRS || (p.mode == ROPE_MG_HALVES ? p.D % 8 == 0 : p.n_rot % 8 == 0);
    const dim3 grid((unsigned) ((waves + 3) / 4));
    if (p.D <= 256) {
        if (vec && p.D == 128) pre_attn_kernel<true, 1, 128><<<grid, 256, 0, g->q>>>(q);
        else if (vec && p.D == 256) pre_attn_kernel<true, 1, 256><<<grid, 256, 0, g->q>>>(q);
        else if (vec) pre_attn_kernel<true, 1, 0><<<grid, 256, 0, g->q>>>(q);
        else pre_attn_kernel<false, 1, 0><<<grid, 256, 0, g->q>>>(q);
    } else {
        if (vec) pre_attn_kernel<true, 2, 0><<<grid, 256, 0, g->q>>>(q);
        else pre_attn_kernel<false, 2, 0><<<grid, 256, 0, g->q>>>(q);
    }
    NS_LAUNCHED(who);
    return 0;
}

inline bool al16(const void* p) { return (uintptr_t) p % 16 == 0; }

}  // namespace

extern "C" {

int ns_q35_qk_norm_rope_pos(ns_gpu* g, const float* src, int64_t ss, int64_t hs, float* dst, int64_t ds, int64_t T, int64_t H, int64_t D,
                            const float* w, float eps, int64_t n_rot, float theta, const int32_t* pos, int64_t s0, int64_t s1, int64_t s2) {
    NS_TRY
    if (T <= 0) return 0;
    if (D % 16 != 0 || D > 512 || n_rot > D || n_rot % 2 || n_rot < 0 || s0 + s1 + s2 <= 0)
        return ns_fail("ns_q35_qk_norm_rope_pos: D a multiple of 16 up to 512, n_rot even and at most D, sections");
    if (!src || !dst || !w || !pos) return ns_fail("ns_q35_qk_norm_rope_pos: a null buffer");
    if (!al16(src) || !al16(dst) || ss % 4 || hs % 4 || ds % 4) return ns_fail("ns_q35_qk_norm_rope_pos: rows 16-byte aligned");
    PreParams p{};
    p.gr[0] = PreGroup{(int) H, src, ss, hs, w, 1, dst, ds, DST_F32, nullptr, 0};
    p.ngr = 1;
    p.T = (int) T; p.D = (int) D; p.mode = ROPE_Q35; p.n_rot = (int) n_rot; p.theta = theta; p.eps = eps;
    p.pos3 = pos; p.s0 = (int) s0; p.s1 = (int) s1; p.s2 = (int) s2;
    return launch_pre(g, p, "ns_q35_qk_norm_rope_pos");
    NS_CATCH
}

int ns_q35_qk_norm_rope(ns_gpu* g, const float* src, int64_t ss, int64_t hs, float* dst, int64_t ds, int64_t T, int64_t H, int64_t D,
                        const float* w, float eps, int64_t n_rot, float theta, int64_t p0) {
    NS_TRY
    if (T <= 0) return 0;
    if (D % 16 != 0 || D > 512 || n_rot > D || n_rot % 2 || n_rot < 0) return ns_fail("ns_q35_qk_norm_rope: D a multiple of 16 up to 512, n_rot even and at most D");
    if (!src || !dst || !w) return ns_fail("ns_q35_qk_norm_rope: a null buffer");
    if (!al16(src) || !al16(dst) || ss % 4 || hs % 4 || ds % 4) return ns_fail("ns_q35_qk_norm_rope: rows 16-byte aligned");
    PreParams p{};
    p.gr[0] = PreGroup{(int) H, src, ss, hs, w, 1, dst, ds, DST_F32, nullptr, 0};
    p.ngr = 1;
    p.T = (int) T; p.D = (int) D; p.mode = ROPE_Q35; p.n_rot = (int) n_rot; p.theta = theta; p.eps = eps; p.p0 = p0;
    return launch_pre(g, p, "ns_q35_qk_norm_rope");
    NS_CATCH
}

int ns_rc_qk_norm_rope(ns_gpu* g, const float* src, int64_t ss, int64_t hs, float* dst, int64_t ds, int64_t T, int64_t H, int64_t D,
                       const float* w, float eps, int rope, float theta, int64_t p0) {
    if (T <= 0) return 0;
    if (D % 16 != 0 || D > 512) return ns_fail("ns_rc_qk_norm_rope: D a multiple of 16");
    // (rotate-half over all D features, or none: the qwen35 form with n_rot = D or 0, the same arithmetic)
    return ns_q35_qk_norm_rope(g, src, ss, hs, dst, ds, T, H, D, w, eps, rope ? D : 0, theta, p0);
}

int ns_q35_rope(ns_gpu* g, const float* src, int64_t ss, int64_t hs, float* dst, int64_t ds, int64_t T, int64_t H, int64_t D, int64_t n_rot,
                float theta, int64_t p0) {
    NS_TRY
    if (T <= 0) return 0;
    if (D % 16 != 0 || D > 512 || n_rot > D || n_rot % 2 || n_rot < 0) return ns_fail("ns_q35_rope: D a multiple of 16 up to 512, n_rot even and at most D");
    if (!src || !dst) return ns_fail("ns_q35_rope: a null buffer");
    if (!al16(src) || !al16(dst) || ss % 4 || hs % 4 || ds % 4) return ns_fail("ns_q35_rope: rows 16-byte aligned");
    PreParams p{};
    p.gr[0] = PreGroup{(int) H, src, ss, hs, nullptr, 1, dst, ds, DST_F32, nullptr, 0};
    p.ngr = 1;
    p.T = (int) T; p.D = (int) D; p.mode = ROPE_Q35; p.n_rot = (int) n_rot; p.theta = theta; p.p0 = p0;
    return launch_pre(g, p, "ns_q35_rope");
    NS_CATCH
}

int ns_mg_qk_norm_rope(ns_gpu* g, const float* x, int64_t xs, float* y, int64_t ys, int64_t T, int64_t H, int64_t D, const float* w, float eps,
                       int rope, float theta, int64_t p0) {
    NS_TRY
    if (T <= 0) return 0;
    if (D % 32 != 0 || D > 512) return ns_fail("ns_mg_qk_norm_rope: D a multiple of 32 up to 512");
    if (rope < 0 || rope > 2) return ns_fail("ns_mg_qk_norm_rope: rope 0 (none), 1 (adjacent pairs) or 2 (halves)");
    if (!x || !y || !w) return ns_fail("ns_mg_qk_norm_rope: a null buffer");
    if (!al16(x) || !al16(y) || xs % 4 || ys % 4) return ns_fail("ns_mg_qk_norm_rope: rows 16-byte aligned");
    PreParams p{};
    p.gr[0] = PreGroup{(int) H, x, xs, D, w, rope != 0, y, ys, DST_F32, nullptr, 0};
    p.ngr = 1;
    p.T = (int) T; p.D = (int) D; p.mode = rope == 0 ? ROPE_NONE : rope == 1 ? ROPE_MG_PAIRS : ROPE_MG_HALVES; p.theta = theta; p.eps = eps; p.p0 = p0;
    return launch_pre(g, p, "ns_mg_qk_norm_rope");
    NS_CATCH
}

int ns_llm_minimaxm3_rope(ns_gpu* g, float* x, int64_t T, int64_t H, int64_t row, int64_t head, int64_t n_rot, int64_t pos0, float base) {
    NS_TRY
    if (n_rot <= 0 || n_rot % 2 || n_rot > head) return ns_fail("ns_llm_minimaxm3_rope: n_rot");
    if (T <= 0 || H <= 0) return 0;
    if (head % 4 || head > 512) return ns_fail("ns_llm_minimaxm3_rope: heads of a multiple of 4 up to 512 floats");
    if (!x) return ns_fail("ns_llm_minimaxm3_rope: a null buffer");
    if (!al16(x) || row % 4) return ns_fail("ns_llm_minimaxm3_rope: rows 16-byte aligned");
    PreParams p{};
    p.gr[0] = PreGroup{(int) H, x, row, head, nullptr, 1, x, row, DST_F32, nullptr, 0};
    p.ngr = 1;
    p.T = (int) T; p.D = (int) head; p.mode = ROPE_MM3; p.n_rot = (int) n_rot; p.ts = powf(base, -2.0f / (float) n_rot); p.p0 = pos0;
    return launch_pre(g, p, "ns_llm_minimaxm3_rope");
    NS_CATCH
}

int ns_mm3s_attn_post(ns_gpu* g, float* q, float* k, const float* v, float* iq, float* ik, const float* qn, const float* kn, const float* iqn,
                      const float* ikn, uint16_t* kc, uint16_t* vc, uint16_t* ic, int64_t H, int64_t G, int64_t IH, int64_t HD, int64_t n_rot,
                      int64_t pos, float base, float eps) {
    NS_TRY
    if (n_rot % 2 || n_rot > HD || n_rot < 0) return ns_fail("ns_mm3s_attn_post: n_rot");
    if (HD % 4 || HD > 512 || H <= 0 || G <= 0 || IH < 0) return ns_fail("ns_mm3s_attn_post: heads of a multiple of 4 up to 512 floats");
    if (!q || !k || !v || !qn || !kn || !kc || !vc || (IH > 0 && (!iq || !ik || !iqn || !ikn || !ic))) return ns_fail("ns_mm3s_attn_post: a null buffer");
    if (!al16(q) || !al16(k) || !al16(v) || (IH > 0 && (!al16(iq) || !al16(ik))) || (uintptr_t) kc % 8 || (uintptr_t) vc % 8 || (IH > 0 && (uintptr_t) ic % 8))
        return ns_fail("ns_mm3s_attn_post: rows 16-byte aligned (half rows 8)");
    PreParams p{};
    p.gr[0] = PreGroup{(int) H, q, 0, HD, qn, 1, q, 0, DST_F32, nullptr, 0};
    p.gr[1] = PreGroup{(int) G, k, 0, HD, kn, 1, k, 0, DST_F32, kc, 0};
    // v: no norm, no rotation; the float32 row is left as it is (written back to itself), the half copy is the store
    p.gr[2] = PreGroup{(int) G, v, 0, HD, nullptr, 0, vc, 0, DST_F16, nullptr, 0};
    p.ngr = 3;
    if (IH > 0) {
        p.gr[3] = PreGroup{(int) IH, iq, 0, HD, iqn, 1, iq, 0, DST_F32, nullptr, 0};
        p.gr[4] = PreGroup{1, ik, 0, HD, ikn, 1, ik, 0, DST_F32, ic, 0};
        p.ngr = 5;
    }
    p.T = 1; p.D = (int) HD; p.mode = n_rot > 0 ? ROPE_MM3 : ROPE_NONE; p.n_rot = (int) n_rot; p.ts = n_rot > 0 ? powf(base, -2.0f / (float) n_rot) : 1.0f;
    p.eps = eps; p.p0 = pos; p.inv_sqrt = 1;
    return launch_pre(g, p, "ns_mm3s_attn_post");
    NS_CATCH
}

int ns_attn_pre_store(ns_gpu* g, int rope, int qt, int kt, int ring, const float* q, int64_t qss, int64_t qhs, void* qo, int64_t qos,
                      const float* k, int64_t kss, int64_t khs, const float* v, int64_t vss, const float* qw, const float* kw, float eps,
                      int64_t n_rot, float theta, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, void* kc, void* vc) {
    NS_TRY
    if (T <= 0) return 0;
    if (D != 64 && D != 128 && D != 256) return ns_fail("ns_attn_pre_store: heads of 64, 128 or 256");
    if (rope < 1 || rope > 3) return ns_fail("ns_attn_pre_store: rope 1 (rotate-half over n_rot), 2 (adjacent pairs) or 3 (halves)");
    if (rope == 1 && (n_rot > D || n_rot % 2 || n_rot < 0)) return ns_fail("ns_attn_pre_store: n_rot even and at most D");
    if (qt < 0 || qt > 2 || kt < 0 || kt > 3) return ns_fail("ns_attn_pre_store: rows of type 0..2, a cache form 0..3");
    if (Hq <= 0 || Hkv <= 0 || cap <= 0 || p0 < 0) return ns_fail("ns_attn_pre_store: heads, a capacity and a position");
    if (!ring && p0 + T > cap) return ns_fail("ns_attn_pre_store: past the cache's capacity");
    if (ring && T > cap) return ns_fail("ns_attn_pre_store: more rows than the ring holds");
    if (!q || !qo || !k || !v || !qw || !kw || !kc || !vc) return ns_fail("ns_attn_pre_store: a null buffer");
    if (!al16(q) || !al16(k) || !al16(v) || qss % 4 || qhs % 4 || kss % 4 || khs % 4 || vss % 4 || (uintptr_t) qo % (qt == 0 ? 16 : 8) || qos % 4 ||
        ((uintptr_t) kc | (uintptr_t) vc) % 8)
        return ns_fail("ns_attn_pre_store: rows 16-byte aligned (16-bit rows and caches 8)");
    PreParams p{};
    p.gr[0] = PreGroup{(int) Hq, q, qss, qhs, qw, 1, qo, qos, qt, nullptr, 0};
    p.gr[1] = PreGroup{(int) Hkv, k, kss, khs, kw, 1, kc, 0, DST_CACHE + kt, nullptr, 0};
    p.gr[2] = PreGroup{(int) Hkv, v, vss, D, nullptr, 0, vc, 0, DST_CACHE + kt, nullptr, 0};
    p.ngr = 3;
    p.T = (int) T; p.D = (int) D; p.mode = rope == 1 ? ROPE_Q35 : rope == 2 ? ROPE_MG_PAIRS : ROPE_MG_HALVES; p.n_rot = (int) n_rot;
    p.theta = theta; p.eps = eps; p.p0 = p0; p.cap = cap; p.ring = ring;
    return launch_pre(g, p, "ns_attn_pre_store");
    NS_CATCH
}

}  // extern "C"
