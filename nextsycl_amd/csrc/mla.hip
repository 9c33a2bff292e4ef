// mla.hip: DeepSeek-style absorbed MLA decode over the latent cache for gfx950, and its neighbours: the absorb (q~ = k_b
// q_nope), the value up-projection (out = v_b u), the latent cache store (RMS norm + YaRN rope) and GLM's q8 latent rows.
//
// The absorbed decode is one dense contraction per cell tile with "the key is the value": every head scores a cell with
// its 512 latent + 64 rope features and then accumulates the same 512 latent features. Per cell: H x (576 + 512) x 2
// flops against 1152 bytes - ~240 flop/byte at H = 128: the kernel is MFMA-bound and is built so that a cell is read
// from HBM once for ALL heads.
//
// Work split: grid (cell split, row group). A work-group of 8 waves owns 128 (row, head) pairs - one decode row's 128
// heads - a wave 16 of them (one 16-row MFMA tile: 72 registers of queries, 128 of accumulators), and a split of the
// cells in 32-cell tiles; short passes of at most 128 rows run 4 waves = 64 pairs a work-group (mla_waves). Half rows go
// global -> LDS directly two tiles ahead into three LDS buffers (the 4-wave form: three ahead into four), one barrier a
// tile; GLM's q8 rows are fetched through registers and widened to half on the way. The tile is shared by the
// work-group's waves. LDS rows are 74 chunks of 16 bytes (72 of data, 2 of padding): rows 32 bytes apart modulo 256 spread both access patterns
// over the banks - 16 rows x 16 bytes of one column (the score product's operand) and 8 rows x 32 bytes (the
// transposing read); both measured at the full LDS rate, where rows a multiple of 128 bytes apart halve the first.
//
// A wave's tile step (transposed orientation: a lane owns one row of each row tile):
//   S^T[cell][row] = C Q^T          A = cache rows from LDS (ds_read_b128), B = absorbed queries, in registers
//   base-2 online softmax in float32 (scale folded in), causal edge masked per row
//   P^T -> half = the B operand of the second product
//   O^T[latent][row] += C^T P^T     A = the same tile through ds_read_b64_tr_b16; 128 float32 accumulators a lane
// Each wave owns its rows outright, so a split's partial {O[L] / l as halfs, m (log2 units), l} goes from registers
// (through LDS, as 512-byte runs) to scratch [row][split]; the splits are merged by a second kernel, and a pass of one
// split writes its rows' results itself.
//
// Reference behaviour kept: kernels/llm/deepseek2/ds2.cpp:139-258 (q~, scores over [latent | rope] x scale, online
// softmax, u = sum p c / sum p, out = v_b u; L 512, R 64, nope = V = 128), :85-112 (cache rows), and
// kernels/llm/glm5next/glm.cpp:1079-1186,1282-1299 (latent-only MLA, q8 rows [16 half scales][512 int8]).
#include "ns_internal.hpp"
#include "ns_mla.h"
#include "attn_common.hpp"
#include "attn_host.hpp"
#include "kv_formats.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>

namespace {

constexpr int MTILE = 32, ML = 512;
// waves a work-group (16 rows each): 8 = 128-row groups; 4 = 64-row groups where a group (the pass's rows, or one row's
// heads under a selection) has at most 128 rows and the pass at most 131072 cells - a decode step of 128 heads then runs
// two groups over half as many cell splits: half the query loads and half the partials, which outweighs a tile loop
// twice as long up to about that length (kernel + merge between events, 4 against 8 waves: 35.5 / 42.9 us at 32768
// cells, 46.3 / 51.9 at 65536, 67.4 / 69.1 at 131072)
constexpr int mla_waves(int64_t group_rows, int64_t cells) { return group_rows <= 128 && cells <= 131072 ? 4 : 8; }
// a split's partial of a row: u_s[512] = O_s / l_s as halfs (the split's own normalized result: bounded by the cache's
// values, so half holds it; a quarter of the float32 form's bytes go to m and l), then m (log2 units), l, 2 of padding
constexpr int MLA_PASS_MAX = 256;    // rows of a prompt a pass of the latent kernel takes at most
constexpr int SEL_DENSE_MAX = 2560;   // cells of a dense row in a selection pass (the reference's bound)
constexpr int PSTRIDE = ML / 2 + 4;   // in floats: 1040 bytes, rows stay 16-byte aligned

struct MlaParams {
    const void* qa;      // [T][H][L + R] absorbed queries
    int qt;              // 0 float32, 1 half
    const uint8_t* cache;
    int T, H;
    int64_t pos0;
    int64_t kbs;         // cells a split
    int ns;
    int flat;            // 1: work-group id = split * nz + row group (passes of fewer than 8 splits)
    float sl2;
    float* part;         // [T * H][ns][PSTRIDE]: {half u_s[512], float m, l, -, -}
    // a row's own cells (GLM's selection): sel_cnt[t] >= 0 -> the pools sel[t K ..][0, sel_cnt[t]) of 4 cells each, then
    // the row's incomplete pool 4 ((p + 1) / 4) .. p; negative or no sel_cnt -> every earlier cell. With sel_cnt a row
    // group holds one row t's heads only (per_t), and the kernel's cell numbering runs over the row's list
    const int32_t* sel;
    const int32_t* sel_cnt;
    int K, per_t;
    int nz;              // row groups
    // a pass of one split needs no merge: the kernel writes its rows' results themselves, u [T * H][512] of type ot
    // (0 float32, 1 half), and the partials are not used
    void* u;
    int ot;
};

typedef uint32_t u4v __attribute__((ext_vector_type(4)));   // a 16-byte chunk in flight (a plain vector: stays in registers)

// floats of a split's partial of a row of LW latents: {half u_s[LW], float m, l, -, -}
constexpr int pstride_of(int LW) { return LW / 2 + 4; }

// LW: latent width (512; 256: GLM's other width, latent-only half rows); R: rope features (64: DeepSeek's [512 | 64] rows;
// 0: GLM's latent-only rows); Q8: GLM's q8 rows
template <int LW, int R, bool Q8, int MW>
__global__ __launch_bounds__(MW * 64, MW == 4 ? 1 : 2) void mla_decode_kernel(const MlaParams p) {
    static_assert(LW == 512 || (LW == 256 && R == 0 && !Q8), "latent rows of 512, or latent-only half rows of 256");
    constexpr int ML = LW, PSTRIDE = pstride_of(LW);     // (inside this kernel the latent width is the template's)
    constexpr int MROWS = MW * 16;
    constexpr int DK = ML + R, KB = DK / 32, DT = ML / 16;
    // chunks / bytes a staged row: the data's chunks + 2 of padding at width 512 (whatever R), so that rows lie an odd
    // multiple of 32 bytes apart modulo 256
    constexpr int RCH = LW == 512 ? 74 : LW / 8 + 2, RSTRIDE = RCH * 16;
    // (a buffer also stages four waves' output rows: 16 rows of 528 bytes each)
    constexpr int TILEB = MTILE * RSTRIDE > 4 * 16 * 528 ? MTILE * RSTRIDE : 4 * 16 * 528;
    constexpr int64_t CROW = Q8 ? ML / 32 * 2 + ML : DK * 2;   // bytes a cache row
    constexpr int CPR = Q8 ? ML / 16 : DK / 8;           // 16-byte loads a cache row
    constexpr int NCH = MTILE * CPR;                     // loads a tile
    constexpr int NLD = (NCH + MW * 64 - 1) / (MW * 64); // loads a thread per tile (the last may be idle)
    // three tile buffers (four under the pipelined step of the 4-wave form), separate arrays: reads of one are then
    // known not to touch a buffer a transfer is still writing
    __shared__ __attribute__((aligned(16))) uint8_t lds0[TILEB];
    __shared__ __attribute__((aligned(16))) uint8_t lds1[TILEB];
    __shared__ __attribute__((aligned(16))) uint8_t lds2[TILEB];
    // (the pipelined step works on two tiles at once - it scores tile it + 1 while it weighs tile it - so with three
    // buffers the tile it requests is the one its own end waits for, and a step lasts one memory latency; the fourth
    // buffer lets a request travel a step longer: the tile loop without its products 12.1 -> 9.3 us at 32768 cells)
    constexpr bool FOUR = MW == 4 && !Q8;
    __shared__ __attribute__((aligned(16))) uint8_t lds3[FOUR ? TILEB : 16];
    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    lds_u8* const B0 = (lds_u8*) lds0;
    lds_u8* const B1 = (lds_u8*) lds1;
    lds_u8* const B2 = (lds_u8*) lds2;
    lds_u8* const B3 = (lds_u8*) lds3;

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 15, g4 = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Work-group ids go round the 8 XCDs (each with its own L2). The row groups of one cell split read the same tiles:
    // they get consecutive ids on one XCD, so that they run side by side and a tile comes from memory once. The grid is
    // padded to 8 splits a round; the padding's work-groups leave at once.
    // (A pass of fewer than 8 splits - many row groups over few cells, a prompt's - would leave XCDs idle that way: its
    // row groups are dealt over the XCDs instead, a split's groups in id order.)
    const int xcd = blockIdx.x % 8, xj = blockIdx.x / 8;
    const int z = p.flat ? blockIdx.x % p.nz : xj % p.nz, split = p.flat ? blockIdx.x / p.nz : (xj / p.nz) * 8 + xcd;
    if (split >= p.ns) return;
    const int rows = p.T * p.H;
    // a row group: 128 consecutive (row, head) pairs of the pass, or (per_t) 128 heads of one row t
    const int zpt = (p.H + MROWS - 1) / MROWS;
    const int tz = p.per_t ? z / zpt : 0;
    const int64_t pz = p.pos0 + tz;
    const int64_t cnt = p.per_t && p.sel_cnt ? p.sel_cnt[tz] : -1;        // pools listed for row tz, or negative: dense
    const int64_t tail0 = 4 * ((pz + 1) / 4);
    // cells the group's last row sees (of its list, if it has one)
    const int64_t n_all = !p.per_t ? p.pos0 + p.T : cnt < 0 ? pz + 1 : 4 * cnt + (pz + 1 - tail0);
    const int64_t jb = (int64_t) split * p.kbs, je = std::min(jb + p.kbs, n_all);
    const int32_t* const selt = cnt >= 0 ? p.sel + (int64_t) tz * p.K : nullptr;
    // cell i of the row's numbering -> the cache's cell
    auto cell = [&](int64_t i) -> int64_t {
        if (!selt) return i;
        return i < 4 * cnt ? 4 * (int64_t) selt[i >> 2] + (i & 3) : tail0 + (i - 4 * cnt);
    };

    // ---- this lane's row
    const int rin = (p.per_t ? z % zpt : z) * MROWS + w * 16 + n;        // within the pass, or within row tz's heads
    const bool live = p.per_t ? rin < p.H : rin < rows;
    const int ri = p.per_t ? tz * p.H + rin : rin;
    const int rr = live ? ri : rows - 1;
    const int64_t hi_r = !live ? -1 : p.per_t ? je - 1 : std::min(p.pos0 + rr / p.H, je - 1);
    s8v qreg[KB];
    auto load_queries = [&]() {
        const int64_t qoff = (int64_t) rr * DK + g4 * 8;
        if (p.qt == 0) {
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                const float4 a = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.qa) + qoff + kb * 32);
                const float4 b = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.qa) + qoff + kb * 32 + 4);
                const float f[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
                for (int i = 0; i < 8; ++i) qreg[kb][i] = live ? to16<false>(f[i]) : (short) 0;
            }
        } else {
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                const s8v raw = *reinterpret_cast<const s8v*>(reinterpret_cast<const uint16_t*>(p.qa) + qoff + kb * 32);
#pragma unroll
                for (int i = 0; i < 8; ++i) qreg[kb][i] = live ? raw[i] : (short) 0;
            }
        }
    };
    float nbr = 0.0f, thr = -INFINITY, l_r = 0.0f;
    const int hi_rel = (int) std::max<int64_t>(std::min<int64_t>(hi_r - jb, (int64_t) 1 << 30), -1);
    f4v o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};

    // ---- tile traffic: chunk id = tid + 512 i -> row id / CPR, piece id % CPR; cells past the split's end are clamped
    // to its last (a valid row; their scores are masked)
    // A tile is staged in two phases (loads H1 and NLD - H1 of a thread) through one small register set, so that the
    // registers a tile in flight takes stay few beside the 200 of the queries and accumulators.
    constexpr int H1 = (NLD + 1) / 2;
    u4v st[H1];
    uint16_t stsc[Q8 ? H1 : 1];
    // (a tile wholly inside the split is read at a wave-uniform address plus a 32-bit lane offset)
    const uint8_t* const split_base = p.cache + jb * CROW;
    const int last_rel = (int) (je - 1 - jb);
    auto fetch = [&](int it_, int i0, int i1) {
        const bool plain = !selt && (it_ + 1) * MTILE - 1 <= last_rel;
        const uint8_t* sp = selt ? p.cache : split_base + (plain ? (int64_t) it_ * MTILE * CROW : 0);
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            if (i < i0 || i >= i1) continue;
            const int id = tid + MW * 64 * i, r = id / CPR, c = id % CPR;
            if (NCH % (MW * 64) != 0 && id >= NCH) continue;
            const int rel = plain ? r : std::min(it_ * MTILE + r, last_rel);
            const uint32_t off = (uint32_t) ((selt ? cell(jb + rel) : (int64_t) rel) * CROW);
            if constexpr (Q8) {
                st[i % H1] = *reinterpret_cast<const u4v*>(sp + off + ML / 32 * 2 + c * 16);
                stsc[i % H1] = *reinterpret_cast<const uint16_t*>(sp + off + 2 * (c / 2));
            } else {
                st[i % H1] = *reinterpret_cast<const u4v*>(sp + off + c * 16);
            }
        }
    };
    auto stash = [&](lds_u8* base, int i0, int i1) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            if (i < i0 || i >= i1) continue;
            const int id = tid + MW * 64 * i, r = id / CPR, c = id % CPR;
            if (NCH % (MW * 64) != 0 && id >= NCH) continue;
            if constexpr (Q8) {
                // 16 int8 x one half scale -> 16 halfs = chunks 2c, 2c + 1; value = half(scale) x q, one rounding to
                // half (the reference widens half(scale) x q in float32: kernels/llm/glm5next/glm.cpp:1116-1124)
                const _Float16 d = __builtin_bit_cast(_Float16, stsc[i % H1]);
                const uint32_t ww[4] = {st[i % H1][0], st[i % H1][1], st[i % H1][2], st[i % H1][3]};
                s8v a, b;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const _Float16 x0 = (_Float16) (short) (int8_t) (ww[e >> 2] >> (8 * (e & 3))) * d;
                    const _Float16 x1 = (_Float16) (short) (int8_t) (ww[2 + (e >> 2)] >> (8 * (e & 3))) * d;
                    a[e] = __builtin_bit_cast(short, x0);
                    b[e] = __builtin_bit_cast(short, x1);
                }
                *reinterpret_cast<__attribute__((address_space(3))) s8v*>(base + r * RSTRIDE + (2 * c) * 16) = a;
                *reinterpret_cast<__attribute__((address_space(3))) s8v*>(base + r * RSTRIDE + (2 * c + 1) * 16) = b;
            } else {
                *reinterpret_cast<__attribute__((address_space(3))) u4v*>(base + r * RSTRIDE + c * 16) = st[i % H1];
            }
        }
    };

    // LDS read addresses as a few lane bases plus compile-time offsets: chunk 8 a + b -> one base a value of b, 128 bytes a
    // step of a.
    //   score operand: row ct 16 + n (g the same for both ct), chunk 4 kb + g4        -> b = 4 (kb & 1) + g4, a = kb >> 1
    //   transposed read: row kk (+ 16: same g), chunk 2 dt + ((n & 3) >> 1), half n & 1 -> b = 2 (dt & 3) + .., a = dt >> 2
    const int kk = g4 * 4 + (n >> 2);
    uint32_t s_rd[2], v_rd[4];
#pragma unroll
    for (int b = 0; b < 2; ++b) s_rd[b] = (uint32_t) (n * RSTRIDE + (b * 4 + g4) * 16);
#pragma unroll
    for (int b = 0; b < 4; ++b) v_rd[b] = (uint32_t) (kk * RSTRIDE + (b * 2 + ((n & 3) >> 1)) * 16 + (n & 1) * 8);

    // Half rows go global -> LDS directly (global_load_lds_dwordx4: no register in between, so a tile can be two tiles
    // ahead of the math at no cost in registers). An instruction's 64 lanes fill 64 consecutive 16-byte units of the
    // buffer: unit u = 74 r + x holds chunk x of row r (the two units of padding fetch the row's last chunk again). A wave
    // issues NDMA instructions a tile (units 64 (MW i + w) + lane; in the last round the waves past the tile's end fetch its
    // last 64 units again, so that every wave has the same count in flight).
    constexpr int NU = MTILE * RCH, NDMA = (NU + MW * 64 - 1) / (MW * 64);
    static_assert(NU % 64 == 0, "whole instructions a tile");
    // (a whole tile of a dense split: lane offsets that do not depend on the tile, worked out once)
    // (the 8-wave form has no registers to spare for them)
    constexpr bool DMA_PRE = MW == 4 && !Q8;
    uint32_t dma_off[DMA_PRE ? NDMA : 1];
    if constexpr (DMA_PRE) {
#pragma unroll
        for (int i = 0; i < NDMA; ++i) {
            const int u0 = std::min(i * MW * 64 + w * 64, NU - 64);
            const int u = u0 + lane, r = u / RCH, c = std::min(u % RCH, CPR - 1);
            dma_off[i] = (uint32_t) (r * CROW + c * 16);
        }
    }
    // (one transfer instruction: 64 lanes x 16 bytes from base + the lane's offset to 1 KiB of LDS at dst, wave-uniform.
    // Written out so that the compiler's wait-count pass does not see a memory instruction that writes LDS: it would put
    // a wait for every outstanding transfer in front of the next LDS read - the tile just requested included, which
    // then never travels under the math. The waits the transfers need are written out at the barriers)
    auto dma16 = [&](const uint8_t* base_, uint32_t off, lds_u8* dst) __attribute__((always_inline)) {
        const uint32_t m = __builtin_amdgcn_readfirstlane((uint32_t) (uintptr_t) dst);
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"                   // (m0 is reserved: nothing of the compiler's lives in it across this)
        asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m), "v"(off), "s"(base_) : "memory", "m0");
#pragma clang diagnostic pop
    };
    auto dma = [&](lds_u8* dst, int it_) {
        const bool plain = !selt && (it_ + 1) * MTILE - 1 <= last_rel;
        if constexpr (DMA_PRE) {
            if (plain) {
                const uint8_t* sp = split_base + (int64_t) it_ * MTILE * CROW;
#pragma unroll
                for (int i = 0; i < NDMA; ++i) {
                    const int u0 = std::min(i * MW * 64 + w * 64, NU - 64);
                    dma16(sp, dma_off[i], dst + u0 * 16);
                }
                return;
            }
        }
        const uint8_t* sp = selt ? p.cache : split_base + (plain ? (int64_t) it_ * MTILE * CROW : 0);
#pragma unroll
        for (int i = 0; i < NDMA; ++i) {
            const int u0 = std::min(i * MW * 64 + w * 64, NU - 64);
            const int u = u0 + lane, r = u / RCH, c = std::min(u % RCH, CPR - 1);
            const int rel = plain ? r : std::min(it_ * MTILE + r, last_rel);
            const uint32_t off = (uint32_t) ((selt ? cell(jb + rel) : (int64_t) rel) * CROW + c * 16);
            dma16(sp, off, dst + u0 * 16);
        }
    };

    // One tile: rd holds it, nx1 / nx2 are the buffers of the next two. Half rows: tile it + 2 is requested before the
    // math and tile it + 1 (requested a tile ago) is waited for after it - by every wave for its own transfers, then
    // the barrier makes them everybody's. q8 rows: tile it + 1 is fetched, widened and written in two phases around
    // the math.
    const int nt = jb < je ? (int) ((je - jb + MTILE - 1) / MTILE) : 0;
    auto step = [&](lds_u8* rd, lds_u8* nx1, lds_u8* nx2, int it) {
        const bool more = it + 1 < nt;
        if constexpr (Q8) {
            if (more) fetch(it + 1, 0, H1);
        } else {
            if (it + 2 < nt) dma(nx2, it + 2);
        }
        // ---- S^T = C Q^T: the two cell tiles' chains alternate, operands read a few steps ahead of their use
        f4v s[2] = {f4v{0.0f, 0.0f, 0.0f, 0.0f}, f4v{0.0f, 0.0f, 0.0f, 0.0f}};
        {
            auto ld = [&](int kb, int ct) {
                return *reinterpret_cast<const __attribute__((address_space(3))) s8v*>(rd + s_rd[kb & 1] + ct * 16 * RSTRIDE + (kb >> 1) * 128);
            };
            constexpr int AHEAD = MW == 4 ? 3 : 1;                 // kb steps (two reads each) in flight
            s8v fa[AHEAD + 1][2];
#pragma unroll
            for (int kb = 0; kb < AHEAD; ++kb) {
                fa[kb][0] = ld(kb, 0);
                fa[kb][1] = ld(kb, 1);
            }
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                if (kb + AHEAD < KB) {
                    fa[(kb + AHEAD) % (AHEAD + 1)][0] = ld(kb + AHEAD, 0);
                    fa[(kb + AHEAD) % (AHEAD + 1)][1] = ld(kb + AHEAD, 1);
                }
                s[0] = mfma16<false>(fa[kb % (AHEAD + 1)][0], qreg[kb], s[0]);
                s[1] = mfma16<false>(fa[kb % (AHEAD + 1)][1], qreg[kb], s[1]);
            }
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * AHEAD, 0);
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                if (kb + AHEAD < KB) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            }
        }
        // ---- softmax of this lane's row, in base-2 exponent units. The reference the weights are taken against (minus
        // it: nbr) moves - and the 128 accumulators are rescaled - only when some score of the wave outgrows it by more
        // than 2^8 (thr; -inf while the row has seen no cell: the first one sets it). Weights may otherwise exceed 1, by
        // at most 2^8: harmless in float32 sums and half operands, and the partial's {O, m, l} stay consistent. The
        // common path has no cross-lane step: l_r is this lane's own share of the row's sum.
        s8v pb;
        {
            float a[8];
            const int hi = hi_rel - it * MTILE;                    // cells 0 .. hi of this tile are the row's
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int j = (e >> 2) * 16 + g4 * 4 + (e & 3);
                a[e] = j <= hi ? __builtin_fmaf(s[e >> 2][e & 3], p.sl2, nbr) : -INFINITY;
            }
            const float amax = fmaxf(fmaxf(fmaxf(a[0], a[1]), fmaxf(a[2], a[3])), fmaxf(fmaxf(a[4], a[5]), fmaxf(a[6], a[7])));
            if (__any(amax > thr)) {
                const float mx = rows_max(amax);
                const bool fresh = thr < 0.0f, nokey = mx == -INFINITY;
                const float delta = fresh ? (nokey ? 0.0f : mx) : fmaxf(mx, 0.0f);
                const float c = fresh ? 1.0f : fast_exp2(-delta);
                l_r *= c;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) o[dt] *= c;
                nbr -= delta;
#pragma unroll
                for (int e = 0; e < 8; ++e) a[e] -= delta;
                thr = (fresh && nokey) ? -INFINITY : 8.0f;
            }
            float sum = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float pv = fast_exp2(a[e]);                   // -inf -> 0
                sum += pv;
                pb[e] = to16<false>(pv);
            }
            l_r += sum;
        }
        if constexpr (Q8) {
            if (more) {
                stash(nx1, 0, H1);
                fetch(it + 1, H1, NLD);
            }
        }
        // ---- O^T += C^T P^T, the transposed reads two steps ahead of their use
        {
            auto ldt = [&](int dt) {
                const lds_u8* src = rd + v_rd[dt & 3] + (dt >> 2) * 128;
                const s4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*) src);
                const s4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*) (src + 16 * RSTRIDE));
                return s8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            };
            constexpr int AHEAD = MW == 4 ? 6 : 2;
            s8v va[AHEAD + 1];
#pragma unroll
            for (int dt = 0; dt < AHEAD; ++dt) va[dt] = ldt(dt);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                if (dt + AHEAD < DT) va[(dt + AHEAD) % (AHEAD + 1)] = ldt(dt + AHEAD);
                o[dt] = mfma16<false>(va[dt % (AHEAD + 1)], pb, o[dt]);
            }
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * AHEAD, 0);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                if (dt + AHEAD < DT) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            }
        }
        if constexpr (Q8) {
            if (more) stash(nx1, H1, NLD);
            __syncthreads();
        } else {
            // this wave's transfers of tile it + 1 are done when at most tile it + 2's are still in flight, and every LDS read
            // it has issued has returned (a wave past the barrier requests a transfer into the buffer this step read); a
            // bare barrier then (the fence of __syncthreads would wait for tile it + 2 as well)
            if (it + 2 < nt) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(NDMA) : "memory");
            else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        }
    };
    // Half rows: the same three parts software-pipelined over the tiles, so that the one wave a SIMD holds keeps its matrix
    // pipe fed while the vector unit works - a tile's step is two straight-line blocks,
    //   1: S^T of tile it + 1 (its buffer landed a step ago)   ||   weights of tile it = exp2(arguments), sum, rounding
    //   2: O^T += C^T P^T of tile it                           ||   exponent arguments of tile it + 1 and their largest
    // then (rarely) the move of the reference, the wait for tile it + 2's transfers (tile it + 3's, requested at the
    // step's head, stay in flight) and the barrier. Past the split's last
    // tile block 1 scores whatever the next buffer holds: every such cell is masked.
    float a_cur[8];
    auto args_of = [&](const f4v (&s)[2], int it, float (&a)[8]) -> float {
        const int hi = hi_rel - it * MTILE;                    // cells 0 .. hi of this tile are the row's
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int j = (e >> 2) * 16 + g4 * 4 + (e & 3);
            a[e] = j <= hi ? __builtin_fmaf(s[e >> 2][e & 3], p.sl2, nbr) : -INFINITY;
        }
        return fmaxf(fmaxf(fmaxf(a[0], a[1]), fmaxf(a[2], a[3])), fmaxf(fmaxf(a[4], a[5]), fmaxf(a[6], a[7])));
    };
    auto regrow = [&](float amax, float (&a)[8]) {
        if (__any(amax > thr)) {
            const float mx = rows_max(amax);
            const bool fresh = thr < 0.0f, nokey = mx == -INFINITY;
            const float delta = fresh ? (nokey ? 0.0f : mx) : fmaxf(mx, 0.0f);
            const float c = fresh ? 1.0f : fast_exp2(-delta);
            l_r *= c;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) o[dt] *= c;
            nbr -= delta;
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] -= delta;
            thr = (fresh && nokey) ? -INFINITY : 8.0f;
        }
    };
    auto scores_of = [&](lds_u8* rd, f4v (&s)[2]) {
        s[0] = s[1] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
        auto ld = [&](int kb, int ct) {
            return *reinterpret_cast<const __attribute__((address_space(3))) s8v*>(rd + s_rd[kb & 1] + ct * 16 * RSTRIDE + (kb >> 1) * 128);
        };
        constexpr int AHEAD = MW == 4 ? 3 : 1;                 // kb steps (two reads each) in flight
        s8v fa[AHEAD + 1][2];
#pragma unroll
        for (int kb = 0; kb < AHEAD; ++kb) {
            fa[kb][0] = ld(kb, 0);
            fa[kb][1] = ld(kb, 1);
        }
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            if (kb + AHEAD < KB) {
                fa[(kb + AHEAD) % (AHEAD + 1)][0] = ld(kb + AHEAD, 0);
                fa[(kb + AHEAD) % (AHEAD + 1)][1] = ld(kb + AHEAD, 1);
            }
            s[0] = mfma16<false>(fa[kb % (AHEAD + 1)][0], qreg[kb], s[0]);
            s[1] = mfma16<false>(fa[kb % (AHEAD + 1)][1], qreg[kb], s[1]);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * AHEAD, 0);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            if (kb + AHEAD < KB) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            if (kb % 2 == 0 && kb < 16) __builtin_amdgcn_sched_group_barrier(0x400, 1, 0);      // an exponential of the tile before
        }
    };
    auto weigh_of = [&](lds_u8* rd, const s8v pb) {
        auto ldt = [&](int dt) {
            const lds_u8* src = rd + v_rd[dt & 3] + (dt >> 2) * 128;
            const s4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*) src);
            const s4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*) (src + 16 * RSTRIDE));
            return s8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        };
        constexpr int AHEAD = MW == 4 ? 6 : 2;
        s8v va[AHEAD + 1];
#pragma unroll
        for (int dt = 0; dt < AHEAD; ++dt) va[dt] = ldt(dt);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            if (dt + AHEAD < DT) va[(dt + AHEAD) % (AHEAD + 1)] = ldt(dt + AHEAD);
            o[dt] = mfma16<false>(va[dt % (AHEAD + 1)], pb, o[dt]);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * AHEAD, 0);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            if (dt + AHEAD < DT) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
    };
    auto pstep = [&](lds_u8* rd, lds_u8* nx1, lds_u8* nx3, int it) {
        if (it + 3 < nt) dma(nx3, it + 3);
        // ---- block 1
        f4v s[2];
        scores_of(nx1, s);
        s8v pb;
        {
            float sum = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float pv = fast_exp2(a_cur[e]);               // -inf -> 0
                sum += pv;
                pb[e] = to16<false>(pv);
            }
            l_r += sum;
        }
        // ---- block 2
        weigh_of(rd, pb);
        const float amax = args_of(s, it + 1, a_cur);
        regrow(amax, a_cur);
        // (the next step's first block reads tile it + 2, requested a step ago: only this step's request may stay out)
        if (it + 3 < nt) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(NDMA) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    if constexpr (Q8) {
        load_queries();
        if (nt > 0) {
            fetch(0, 0, H1);
            stash(B0, 0, H1);
            fetch(0, H1, NLD);
            stash(B0, H1, NLD);
        }
        __syncthreads();
        for (int it = 0; it < nt; it += 3) {
            step(B0, B1, B2, it);
            if (it + 1 >= nt) break;
            step(B1, B2, B0, it + 1);
            if (it + 2 >= nt) break;
            step(B2, B0, B1, it + 2);
        }
    } else if constexpr (MW == 8) {
        // (two waves a SIMD overlap each other; the pipelined form's extra live registers would spill at 256 a wave)
        if (nt > 0) dma(B0, 0);
        if (nt > 1) dma(B1, 1);
        load_queries();
        if (nt > 1) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(NDMA) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        for (int it = 0; it < nt; it += 3) {
            step(B0, B1, B2, it);
            if (it + 1 >= nt) break;
            step(B1, B2, B0, it + 1);
            if (it + 2 >= nt) break;
            step(B2, B0, B1, it + 2);
        }
    } else {
        // the first two tiles are on their way before the queries are loaded, the third behind them
        if (nt > 0) dma(B0, 0);
        if (nt > 1) dma(B1, 1);
        load_queries();
        if (nt > 2) dma(B2, 2);
        if (nt > 2) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(NDMA) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (nt > 0) {
            f4v s[2];
            scores_of(B0, s);
            const float amax = args_of(s, 0, a_cur);
            regrow(amax, a_cur);
        }
        if constexpr (FOUR) {
            for (int it = 0; it < nt; it += 4) {
                pstep(B0, B1, B3, it);
                if (it + 1 >= nt) break;
                pstep(B1, B2, B0, it + 1);
                if (it + 2 >= nt) break;
                pstep(B2, B3, B1, it + 2);
                if (it + 3 >= nt) break;
                pstep(B3, B0, B2, it + 3);
            }
        }
    }

    // ---- the split's partial {u_s = O / l as halfs, m, l}. A lane holds latents 16 dt + 4 g4 .. + 3 of its row: the
    // wave's 16 x 512 block goes through LDS (the tile buffers, free now: the loop ended on a barrier with every transfer
    // landed), half of the latents at a time, so that it leaves as 512-byte runs of a row
    const float l_row = rows_sum(l_r);
    const float m_r = thr < 0.0f ? -INFINITY : -nbr;
    const float inv_l = l_row > 0.0f ? 1.0f / l_row : 0.0f;
    if (p.ns == 1 && p.u) {
        // ---- one split: the rows' results, through the same staging (512 bytes a row and pass: 256 halfs, or 128 floats).
        // (a dense row of a selection pass past the length such passes are sized for comes out as NaNs, not as a
        // plausible wrong answer)
        constexpr int OROW = 512 + 16;
        lds_u8* const ob = (w < 4 ? B0 : B1) + (w & 3) * 16 * OROW;
        typedef _Float16 h4v __attribute__((ext_vector_type(4)));
        const float sc = n_all > p.kbs ? __builtin_nanf("") : inv_l;
        const int64_t rowb = p.ot == 0 ? ML * 4 : ML * 2;
        const int passes = (int) (rowb / 512), dpp = DT / passes;     // passes of 512 bytes over a row's latents, 16-latent tiles a pass
        for (int hp = 0; hp < passes; ++hp) {
#pragma unroll
            for (int d2 = 0; d2 < 16; ++d2) {
                if (d2 < dpp) {
                    // (o indexed through a constant-trip loop: the accumulators stay in registers)
                    f4v v = o[0];
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) v = dt == hp * dpp + d2 ? o[dt] : v;
                    v = v * sc;
                    if (p.ot == 0) {
                        *reinterpret_cast<__attribute__((address_space(3))) f4v*>(ob + n * OROW + (d2 * 16 + g4 * 4) * 4) = v;
                    } else {
                        const h4v h = {(_Float16) v[0], (_Float16) v[1], (_Float16) v[2], (_Float16) v[3]};
                        *reinterpret_cast<__attribute__((address_space(3))) h4v*>(ob + n * OROW + (d2 * 16 + g4 * 4) * 2) = h;
                    }
                }
            }
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const int id = c * 64 + lane, r = id >> 5, piece = id & 31;
                const int rg = (p.per_t ? z % zpt : z) * MROWS + w * 16 + r;
                const bool ok = p.per_t ? rg < p.H : rg < rows;
                const int64_t rrow = p.per_t ? (int64_t) tz * p.H + rg : rg;
                const u4v x = *reinterpret_cast<const __attribute__((address_space(3))) u4v*>(ob + r * OROW + piece * 16);
                if (ok) *reinterpret_cast<u4v*>(reinterpret_cast<uint8_t*>(p.u) + rrow * rowb + hp * 512 + piece * 16) = x;
            }
        }
        return;
    }
    {
        constexpr int OROW = 256 * 2 + 16;                        // bytes a staged row of 256 halfs, padded
        lds_u8* const ob = (w < 4 ? B0 : B1) + (w & 3) * 16 * OROW;   // 4 waves x 8,448 bytes in each of the first two buffers
        static_assert(4 * 16 * OROW <= TILEB, "the staging fits a tile buffer");
        typedef _Float16 h4v __attribute__((ext_vector_type(4)));
        float* const prow = p.part + (int64_t) split * PSTRIDE;
#pragma unroll
        for (int hp = 0; hp < ML / 256; ++hp) {
#pragma unroll
            for (int d2 = 0; d2 < 16; ++d2) {
                const f4v v = o[hp * 16 + d2] * inv_l;
                const h4v h = {(_Float16) v[0], (_Float16) v[1], (_Float16) v[2], (_Float16) v[3]};
                *reinterpret_cast<__attribute__((address_space(3))) h4v*>(ob + n * OROW + (d2 * 16 + g4 * 4) * 2) = h;
            }
            // the wave reads back its own rows only: no barrier (the LDS queue keeps a wave's accesses in order)
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const int id = c * 64 + lane, r = id >> 5, piece = id & 31;      // 32 pieces of 16 bytes a row's half
                const int rg = (p.per_t ? z % zpt : z) * MROWS + w * 16 + r;
                const bool ok = p.per_t ? rg < p.H : rg < rows;
                const int64_t rrow = p.per_t ? (int64_t) tz * p.H + rg : rg;
                const u4v x = *reinterpret_cast<const __attribute__((address_space(3))) u4v*>(ob + r * OROW + piece * 16);
                if (ok) *reinterpret_cast<u4v*>(reinterpret_cast<uint8_t*>(prow + rrow * p.ns * PSTRIDE) + hp * 512 + piece * 16) = x;
            }
        }
        if (live && g4 == 0) {
            float* pr = prow + (int64_t) ri * p.ns * PSTRIDE;
            // (a row with more cells than the launch has splits for - a dense row of a selection pass past the length such
            // passes are sized for - must not come out looking right: its partials' maxima are not numbers)
            pr[ML / 2] = n_all > (int64_t) p.ns * p.kbs ? __builtin_nanf("") : m_r;
            pr[ML / 2 + 1] = l_row;
        }
    }
}

// the splits of a row merged: u = sum_s u_s w_s / sum_s w_s, w_s = l_s 2^(m_s - M). Two work-groups of 256 threads a row,
// 256 latents each: a thread sums 4 latents (one 8-byte load a split) over every fourth split, then the four phases are
// added in a fixed order. A thread's first 32 loads are requested before anything else, so that they travel while the
// splits' (m, l) are fetched and turned into weights: one memory latency a row instead of three.
template <int LW, int QT>
__global__ __launch_bounds__(256) void mla_merge_kernel(const float* __restrict__ part, int ns, void* __restrict__ u) {
    constexpr int ML = LW, PSTRIDE = pstride_of(LW);     // (two work-groups a row at width 512, one at 256)
    __shared__ float wsh[1024];
    __shared__ float red[8];
    __shared__ f4v ph[256];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const float* pr = part + row * ns * PSTRIDE;
    const int quad = tid & 63, phase = tid >> 6;
    const int lat = blockIdx.y * 256 + quad * 4;
    typedef _Float16 h4v __attribute__((ext_vector_type(4)));
    constexpr int CH = 32;                                         // loads a thread keeps in flight
    h4v hv[CH];
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int sp = phase + 4 * i;
        hv[i] = sp < ns ? *reinterpret_cast<const h4v*>(reinterpret_cast<const _Float16*>(pr + sp * PSTRIDE) + lat) : h4v{0, 0, 0, 0};
    }
    // (m, l) of up to 1024 splits: 4 a thread
    float mv[4], lv[4];
    float mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int sp = tid + 256 * k;
        const float2 ml = sp < ns ? *reinterpret_cast<const float2*>(pr + sp * PSTRIDE + ML / 2) : float2{-INFINITY, 0.0f};
        mv[k] = ml.x;
        lv[k] = ml.y;
        mx = fmaxf(mx, ml.x);                                      // (a marked split's NaN does not take part in the maximum)
    }
    mx = wave_max(mx);
    if (lane == 0) red[wv] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float ls = 0.0f;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int sp = tid + 256 * k;
        const float wgt = mv[k] == -INFINITY ? 0.0f : lv[k] * fast_exp2(mv[k] - mx);
        if (sp < ns) wsh[sp] = wgt;
        ls += wgt;
    }
    ls = wave_sum(ls);
    if (lane == 0) red[4 + wv] = ls;
    __syncthreads();
    const float L = (red[4] + red[5]) + (red[6] + red[7]);
    f4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int sp = phase + 4 * i;
        if (sp < ns) acc += f4v{(float) hv[i][0], (float) hv[i][1], (float) hv[i][2], (float) hv[i][3]} * wsh[sp];
    }
#pragma unroll 8
    for (int sp = phase + 4 * CH; sp < ns; sp += 4) {
        const h4v h = *reinterpret_cast<const h4v*>(reinterpret_cast<const _Float16*>(pr + sp * PSTRIDE) + lat);
        acc += f4v{(float) h[0], (float) h[1], (float) h[2], (float) h[3]} * wsh[sp];
    }
    ph[tid] = acc;
    __syncthreads();
    if (phase == 0) {
        const f4v t = ((ph[quad] + ph[64 + quad]) + ph[128 + quad]) + ph[192 + quad];
#pragma unroll
        for (int i = 0; i < 4; ++i) store_o<QT>(u, row * ML + lat + i, L > 0.0f ? t[i] / L : L != L ? L : 0.0f);      // (a marked row stays NaN)
    }
}

// q~ = k_b q_nope: qa [T][H][L + R] = [k_b[h] q[t][h][:nope] | q[t][h][nope:]]; four work-groups a (row, head), a wave 32
// latent rows of k_b four at a time (all 8 loads requested before the first is used): 16 lanes a row (16 bytes each: the wave's load is 1 KiB of consecutive memory), a
// lane's 8 products summed in feature order, the 16 partial sums through DPP (kernels/llm/deepseek2/ds2.cpp:176-184)
__global__ __launch_bounds__(256) void mla_absorb_kernel(const float* __restrict__ q, const uint16_t* __restrict__ kb, uint16_t* __restrict__ qa,
                                                         int64_t H) {
    constexpr int NOPE = 128, R = 64;
    const int64_t th = blockIdx.x, h = th % H;
    const int part = blockIdx.y;                                   // a quarter of the latent rows a work-group
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, sub = lane & 15, rsel = lane >> 4;
    float qv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) qv[e] = q[th * (NOPE + R) + sub * 8 + e];
    const int r0 = part * 128 + w * 32 + rsel;
    const uint16_t* wbase = kb + ((size_t) h * ML + r0) * NOPE + sub * 8;
    uint4 x[8];
#pragma unroll
    for (int it = 0; it < 8; ++it) x[it] = *reinterpret_cast<const uint4*>(wbase + (size_t) it * 4 * NOPE);     // all in flight at once
#pragma unroll
    for (int it = 0; it < 8; ++it) {
        const uint32_t ww[4] = {x[it].x, x[it].y, x[it].z, x[it].w};
        float a = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) a += f16_to_f32((uint16_t) (ww[e >> 1] >> (16 * (e & 1)))) * qv[e];
        a = row16_sum(a);
        if (sub == 0) qa[th * (ML + R) + r0 + it * 4] = (uint16_t) to16<false>(a);
    }
    if (part == 0 && tid < R) qa[th * (ML + R) + ML + tid] = (uint16_t) to16<false>(q[th * (NOPE + R) + NOPE + tid]);
}

// out [T][H][V] = v_b u: four work-groups a (row, head), a wave a value row at a time (kernels/llm/deepseek2/ds2.cpp:237-255)
__global__ __launch_bounds__(256) void mla_vb_kernel(const float* __restrict__ u, const uint16_t* __restrict__ vb, float* __restrict__ out,
                                                     int64_t H) {
    constexpr int V = 128;
    __shared__ float us[ML];
    const int64_t th = blockIdx.x, h = th % H;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    for (int i = tid; i < ML; i += 256) us[i] = u[th * ML + i];
    __syncthreads();
    // a quarter of the value rows a work-group, 8 a wave: their loads all requested before the first is used
    const int r0 = blockIdx.y * 32 + w * 8;
    uint4 x[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = reinterpret_cast<const uint4*>(vb + ((size_t) h * V + r0 + i) * ML)[lane];
    float uv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) uv[e] = us[lane * 8 + e];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t ww[4] = {x[i].x, x[i].y, x[i].z, x[i].w};
        float a = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) a += f16_to_f32((uint16_t) (ww[e >> 1] >> (16 * (e & 1)))) * uv[e];
        a = wave_sum(a);
        if (lane == 0) out[th * V + r0 + i] = a;
    }
}

// ---- k_b / v_b as the model file stores them: Q6_K rows of 512 (two blocks of 210 bytes: ql [128], qh [64], int8 scales
// [16], a half d), per head its 128 k rows and then its 128 v rows (kernels/llm/deepseek2/ds2.cpp:117-134). A lane owns the
// columns 8 lane .. 8 lane + 7 of a row: eight consecutive values of one 32-value group, so one scale, eight ql bytes (low
// or high nibbles) and eight qh bytes (two bits each). value = d x scale x (q - 32), the products in that order, in float32.
__device__ __forceinline__ void q6k_cols8(const uint8_t* row, int lane, float (&v)[8]) {
    const uint8_t* b = row + (lane >> 5) * 210;                   // the row's block: columns 0..255 / 256..511
    const int j = (lane & 31) * 8, n = j >> 7, gq = (j & 127) >> 5, l0 = j & 31;
    const uint16_t* ql = reinterpret_cast<const uint16_t*>(b + 64 * n + (gq & 1) * 32 + l0);       // (blocks are 2-byte aligned)
    const uint16_t* qh = reinterpret_cast<const uint16_t*>(b + 128 + 32 * n + l0);
    const float ds = f16_to_f32(*reinterpret_cast<const uint16_t*>(b + 208)) * (float) (int8_t) b[192 + 8 * n + 2 * gq + (l0 >> 4)];
    const int shift = 2 * gq;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int lb = (ql[e >> 1] >> (8 * (e & 1))) & 0xFF, hb = (qh[e >> 1] >> (8 * (e & 1))) & 0xFF;
        const int lo = gq < 2 ? (lb & 0xF) : (lb >> 4);
        v[e] = ds * (float) ((lo | (((hb >> shift) & 3) << 4)) - 32);
    }
}

// q~ = sum_i q_nope[i] k_i over a head's 128 Q6_K k rows: a work-group a (row, head), a wave every fourth k row, a lane 8
// columns; the four waves' sums added in wave order (kernels/llm/deepseek2/ds2.cpp:157-173)
__global__ __launch_bounds__(256) void mla_absorb_q6k_kernel(const float* __restrict__ q, const uint8_t* __restrict__ kvb, uint16_t* __restrict__ qa,
                                                             int64_t H) {
    constexpr int NOPE = 128, R = 64, V = 128, ROWB = 420;
    __shared__ float part[4][ML];
    const int64_t th = blockIdx.x, h = th % H;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const float* qr = q + th * (NOPE + R);
    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    for (int i = w; i < NOPE; i += 4) {
        float v[8];
        q6k_cols8(kvb + ((size_t) h * (NOPE + V) + i) * ROWB, lane, v);
        const float qi = qr[i];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += qi * v[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) part[w][lane * 8 + e] = acc[e];
    __syncthreads();
    for (int c = tid; c < ML; c += 256) qa[th * (ML + R) + c] = (uint16_t) to16<false>(((part[0][c] + part[1][c]) + part[2][c]) + part[3][c]);
    if (tid < R) qa[th * (ML + R) + ML + tid] = (uint16_t) to16<false>(qr[NOPE + tid]);
}

// out [T][H][V] = v_b u over a head's 128 Q6_K v rows: a wave a value row at a time (kernels/llm/deepseek2/ds2.cpp:237-246)
__global__ __launch_bounds__(256) void mla_vb_q6k_kernel(const float* __restrict__ u, const uint8_t* __restrict__ kvb, float* __restrict__ out,
                                                         int64_t H) {
    constexpr int NOPE = 128, V = 128, ROWB = 420;
    const int64_t th = blockIdx.x, h = th % H;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    float uv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) uv[e] = u[th * ML + lane * 8 + e];
    for (int r = (int) blockIdx.y * 32 + w; r < (int) blockIdx.y * 32 + 32; r += 4) {
        float v[8];
        q6k_cols8(kvb + ((size_t) h * (NOPE + V) + NOPE + r) * ROWB, lane, v);
        float a = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) a += v[e] * uv[e];
        a = wave_sum(a);
        if (lane == 0) out[th * V + r] = a;
    }
}

// ggml's rope_yarn angle of pair i0 (kernels/llm/deepseek2/ds2.cpp:15-34): the angle by repeated products, as it does
__device__ float yarn_ramp(float low, float high, int i0) {
    const float y = ((float) (i0 / 2) - low) / fmaxf(0.001f, high - low);
    return 1.0f - fminf(1.0f, fmaxf(0.0f, y));
}
__device__ void yarn_cs(float pos, int i0, int n_dims, float freq_base, float freq_scale, float ext_factor, float mscale, float corr0, float corr1,
                        float& c, float& s) {
    const float theta_scale = powf(freq_base, -2.0f / (float) n_dims);
    float theta_extrap = pos;
    for (int k = 0; k < i0 / 2; ++k) theta_extrap *= theta_scale;
    const float theta_interp = freq_scale * theta_extrap;
    float theta = theta_interp;
    if (ext_factor != 0.0f) {
        const float ramp_mix = yarn_ramp(corr0, corr1, i0) * ext_factor;
        theta = theta_interp * (1 - ramp_mix) + theta_extrap * ramp_mix;
    }
    c = cosf(theta) * mscale;
    s = sinf(theta) * mscale;
}

// the latent cache's rows pos0..: [RMSnorm(kv[:L]) w | YaRN-rope(kv[L:L+R])] as half; a work-group a row
__global__ __launch_bounds__(256) void ds2_kv_store_kernel(const float* __restrict__ kv, const float* __restrict__ wgt, float eps,
                                                           uint16_t* __restrict__ cache, int64_t L, int64_t R, int64_t pos0, float freq_base,
                                                           float freq_scale, float ext_factor, float mscale, float corr0, float corr1) {
    // the sum of squares in float64 (every product exact, the sum good to 1e-16: whatever the order of the additions, its
    // rounding to float32 is the same number) - the normalized half of a row is then the same bits on any machine
    __shared__ double red[256];
    const int64_t t = blockIdx.x;
    const int tid = threadIdx.x;
    const float* xr = kv + t * (L + R);
    double ss = 0.0;
    for (int64_t i = tid; i < L; i += 256) ss += (double) xr[i] * (double) xr[i];
    red[tid] = ss;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
        if (tid < o) red[tid] += red[tid + o];
        __syncthreads();
    }
    // (the quotient, the root and the reciprocal through float64 and back: each is then the correctly rounded float32
    // result whatever the compiler makes of a float32 division or square root)
    const float arg = (float) ((double) (float) red[0] / (double) (float) L) + eps;
    const float root = (float) sqrt((double) arg);
    const float inv = (float) (1.0 / (double) root);
    uint16_t* o = cache + (pos0 + t) * (L + R);
    // (the float32 product passes through a register of its own: left to itself the compiler folds the last multiply
    // into the conversion - one rounding to half where the cache's rule has two)
    for (int64_t i = tid; i < L; i += 256) {
        float y = xr[i] * inv * wgt[i];
        asm volatile("" : "+v"(y));
        o[i] = f32_to_f16(y);
    }
    for (int64_t i = tid; i < R / 2; i += 256) {
        const int i0 = (int) (2 * i);
        float c, s;
        yarn_cs((float) (pos0 + t), i0, (int) R, freq_base, freq_scale, ext_factor, mscale, corr0, corr1, c, s);
        const float x0 = xr[L + i0], x1 = xr[L + i0 + 1];
        o[L + i0] = f32_to_f16(x0 * c - x1 * s);
        o[L + i0 + 1] = f32_to_f16(x0 * s + x1 * c);
    }
}

// YaRN rotary positions in place on the rotated part of every head of x (adjacent pairs), a copy of that part to out
// where given; a thread a (row, head, pair)
__global__ __launch_bounds__(256) void ds2_rope_kernel(float* __restrict__ x, int64_t T, int64_t H, int64_t row, int64_t head, int64_t off, int64_t n_dims,
                                                       int64_t pos0, float freq_base, float freq_scale, float ext_factor, float mscale, float corr0,
                                                       float corr1, float* __restrict__ out, int64_t out_row, int64_t out_head) {
    const int64_t pairs = n_dims / 2, gi = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (gi >= T * H * pairs) return;
    const int64_t i = gi % pairs, h = (gi / pairs) % H, t = gi / (pairs * H);
    const int i0 = (int) (2 * i);
    float c, s;
    yarn_cs((float) (pos0 + t), i0, (int) n_dims, freq_base, freq_scale, ext_factor, mscale, corr0, corr1, c, s);
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

// GLM's q8 latent rows: a wave a row, a lane... 16 lanes a row, a lane a block of 32: the scale rounded to half BEFORE it
// divides, clamp to +-127 (kernels/llm/glm5next/glm.cpp:1282-1299)
__global__ __launch_bounds__(256) void to_q8row_kernel(const float* __restrict__ x, uint8_t* __restrict__ y, int64_t n) {
    const int64_t gi = (int64_t) blockIdx.x * 256 + threadIdx.x, r = gi / 16;
    const int b = (int) (gi % 16);
    if (r >= n) return;
    const float* xr = x + r * ML + b * 32;
    float v[32], amax = 0.0f;
#pragma unroll
    for (int e = 0; e < 32; e += 4) {
        const float4 f = *reinterpret_cast<const float4*>(xr + e);
        v[e] = f.x; v[e + 1] = f.y; v[e + 2] = f.z; v[e + 3] = f.w;
    }
#pragma unroll
    for (int e = 0; e < 32; ++e) amax = fmaxf(amax, fabsf(v[e]));
    const uint16_t dh = f32_to_f16(amax / 127.0f);
    const float d = f16_to_f32(dh), inv = d > 0.0f ? 1.0f / d : 0.0f;
    uint8_t* row = y + r * (ML / 32 * 2 + ML);
    reinterpret_cast<uint16_t*>(row)[b] = dh;
    uint32_t* qs = reinterpret_cast<uint32_t*>(row + 32 + b * 32);
#pragma unroll
    for (int e = 0; e < 32; e += 4) {
        uint32_t wv = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) wv |= (uint32_t) (uint8_t) (int8_t) fminf(127.0f, fmaxf(-127.0f, roundf(v[e + k] * inv))) << (8 * k);
        qs[e / 4] = wv;
    }
}

// float32 -> half, 8 values a thread (a float32 latent cache's rows on their way to the latent kernel)
__global__ __launch_bounds__(256) void to_half_kernel(const float* __restrict__ x, uint16_t* __restrict__ y, int64_t n8) {
    const int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (i >= n8) return;
    const float4 a = reinterpret_cast<const float4*>(x)[2 * i], b = reinterpret_cast<const float4*>(x)[2 * i + 1];
    typedef uint16_t us8v __attribute__((ext_vector_type(8)));
    const us8v h = {f32_to_f16(a.x), f32_to_f16(a.y), f32_to_f16(a.z), f32_to_f16(a.w), f32_to_f16(b.x), f32_to_f16(b.y), f32_to_f16(b.z), f32_to_f16(b.w)};
    reinterpret_cast<us8v*>(y)[i] = h;
}

// out [n][512] half = the q8 latent rows idx[i] of src widened: half(scale x q), one rounding (the product is exact in
// float32); a thread 8 values (kernels/llm/glm5next/glm.cpp:1301-1325)
__global__ __launch_bounds__(256) void gather_q8_h_kernel(const uint8_t* __restrict__ src, const int32_t* __restrict__ idx, uint16_t* __restrict__ out,
                                                          int64_t n) {
    const int64_t gi = (int64_t) blockIdx.x * 256 + threadIdx.x, r = gi / 64;
    const int c = (int) (gi % 64);
    if (r >= n) return;
    const uint8_t* row = src + (int64_t) idx[r] * (ML / 32 * 2 + ML);
    const float d = f16_to_f32(reinterpret_cast<const uint16_t*>(row)[c / 4]);
    const uint2 qv = *reinterpret_cast<const uint2*>(row + 32 + c * 8);
    const uint32_t ww[2] = {qv.x, qv.y};
    typedef uint16_t us8v __attribute__((ext_vector_type(8)));
    us8v h;
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = f32_to_f16(d * (float) (int8_t) (ww[e >> 2] >> (8 * (e & 3))));
    reinterpret_cast<us8v*>(out)[r * 64 + c] = h;
}

// ---- host side --------------------------------------------------------------------------------------------------------

int64_t mla_target_wgs() {
    const int64_t v = ns_tune_get(NS_TUNE_MLA_WGS);
    return v > 0 ? v : 256;
}
// cells a split: ~mla_target_wgs() work-groups over the pass, whole 32-cell tiles, at least 2 tiles. A CU holds one
// work-group and a split's row groups sit on one XCD (an eighth of the places), splits dealt round the XCDs: 3 row groups
// x 86 splits are 11 splits = 33 work-groups an XCD with 32 places - two rounds, the second all but empty, and a round
// that is nearly empty costs as much as a full one. Where the rule's count fills its rounds to less than 85 % the count is
// chosen by cost instead: in units of a tile step a work-group costs its tiles + 5 (its queries, its first tile's latency,
// its partials' stores) and the merge 0.032 a partial of a row group; the count whose rounds and merge add up to the least
int64_t mla_kbs(int64_t cells, int64_t groups, bool lists = false) {
    const int64_t t = mla_target_wgs(), want = (cells * groups + t - 1) / t;
    const int64_t kbs = std::max<int64_t>(2 * MTILE, (want + MTILE - 1) / MTILE * MTILE), ns0 = (cells + kbs - 1) / kbs;
    // (rounds: fewer than 8 splits deal their row groups over the whole chip)
    auto rounds_of = [&](int64_t ns) { return ns < 8 || t < 8 ? (ns * groups + t - 1) / t : ((ns + 7) / 8 * groups + t / 8 - 1) / (t / 8); };
    // (rows with cell lists of their own, splits of fewer than 12 tiles: mostly their fixed cost, and a second round's few
    // work-groups run beside the first's last - the plain rule stands: 12 rows' 2051 listed cells x 128 heads 48 us, by
    // cost 54)
    if (100 * ns0 * groups >= 85 * rounds_of(ns0) * t || ns0 * groups <= t / 2 || (lists && kbs < 12 * MTILE)) return kbs;
    const int64_t tiles = (cells + MTILE - 1) / MTILE, most = std::max<int64_t>(1, std::min<int64_t>(tiles / 2, 4 * t));
    int64_t best = 1;
    double cost = 0.0;
    for (int64_t ns = 1; ns <= most; ++ns) {
        const int64_t len = (tiles + ns - 1) / ns;
        const double c = (double) (rounds_of(ns) * (len + 5)) + 0.032 * (double) (groups * ns);
        if (ns == 1 || c < cost) best = ns, cost = c;
    }
    const int64_t per = (cells + best - 1) / best;
    return std::max<int64_t>(2 * MTILE, (per + MTILE - 1) / MTILE * MTILE);
}

int mla_latent(ns_gpu* g, const char* who, int qt, int ot, int R, bool q8, const void* qa, const void* cache, void* u, int64_t T, int64_t H,
               int64_t pos0, float scale, float* scratch, size_t scratch_floats, const int32_t* sel = nullptr, const int32_t* sel_cnt = nullptr,
               int64_t K = 0, int LW = 512) {
    const std::string w(who);
    if (T <= 0) return 0;
    if (LW != 512 && (LW != 256 || R != 0 || q8)) return ns_fail(w + ": latent rows of 512, or latent-only half rows of 256");
    const int64_t PSTRIDE = pstride_of(LW);
    if (H <= 0 || pos0 < 0) return ns_fail(w + ": heads and a position");
    if (T > MLA_PASS_MAX) return ns_fail(w + ": more rows than a pass holds");
    if (!qa || !cache || !u || !scratch) return ns_fail(w + ": a null buffer");
    if (((uintptr_t) qa | (uintptr_t) cache | (uintptr_t) scratch) % 16) return ns_fail(w + ": buffers 16-byte aligned");
    if (!(scale > 0.0f)) return ns_fail(w + ": a positive scale");
    NS_HIP(hipSetDevice(g->dev));
    // With a selection (sel_cnt on the device) a row group holds one row's heads; a row's cell count is only known there:
    // at most 4 K + 3 listed cells, or - where its count is negative - every earlier cell, which the reference allows up
    // to 2,560 tokens only: its kernel keeps a row's scores in 2,560 floats of local memory, and the indexer lists pools
    // past that (kernels/llm/glm5next/glm.cpp:1062-1067, 1085, 1258, 1274). The pass is sized for that many cells; a dense
    // row beyond it comes out as NaNs (the kernel marks it), not as a plausible wrong answer.
    const bool per_t = sel_cnt != nullptr;
    if (per_t && (!sel || K < 0 || K > (int64_t) 1 << 24)) return ns_fail(w + ": a selection has cell pools and their count");
    if ((pos0 + T) * (int64_t) (q8 ? 544 : (LW + R) * 2) >= (int64_t) 1 << 32 && per_t) return ns_fail(w + ": a selection over a cache past 4 GiB");
    const int64_t rows = T * H;
    const int MW = mla_waves(per_t ? H : rows, pos0 + T), MROWS = MW * 16;
    const int64_t nz = per_t ? T * ((H + MROWS - 1) / MROWS) : (rows + MROWS - 1) / MROWS;
    const int64_t listed = 4 * K + 3, cells = per_t ? std::max(listed, std::min<int64_t>(pos0 + T, SEL_DENSE_MAX)) : pos0 + T;
    int64_t kbs = mla_kbs(cells, nz, per_t);
    int64_t ns = (cells + kbs - 1) / kbs;
    // a caller's scratch may be smaller than the rule asks (the library's own, for the reference-named entry points):
    // fewer, longer splits then
    while ((size_t) (rows * ns * PSTRIDE) > scratch_floats && ns > 1) {
        kbs *= 2;
        ns = (cells + kbs - 1) / kbs;
    }
    if ((size_t) (rows * ns * PSTRIDE) > scratch_floats) return ns_fail(w + ": scratch too small");
    if (ns > 1024) return ns_fail(w + ": more cell splits than the merge holds");
    MlaParams p{};
    p.qa = qa;
    p.qt = qt;
    p.cache = (const uint8_t*) cache;
    p.T = (int) T;
    p.H = (int) H;
    p.pos0 = pos0;
    p.kbs = kbs;
    p.ns = (int) ns;
    p.sl2 = scale * 1.4426950408889634f;
    p.part = scratch;
    p.sel = sel;
    p.sel_cnt = sel_cnt;
    p.K = (int) K;
    p.per_t = per_t;
    p.nz = (int) nz;
    p.flat = ns < 8;
    p.u = ns == 1 ? u : nullptr;
    p.ot = ot;
    dim3 grid((unsigned) (p.flat ? ns * nz : (ns + 7) / 8 * 8 * nz));
    if (ns_profile_mark(g, 0)) return -1;
    if (MW == 4) {
        if (LW == 256) mla_decode_kernel<256, 0, false, 4><<<grid, 256, 0, g->q>>>(p);
        else if (q8) mla_decode_kernel<512, 0, true, 4><<<grid, 256, 0, g->q>>>(p);
        else if (R == 64) mla_decode_kernel<512, 64, false, 4><<<grid, 256, 0, g->q>>>(p);
        else mla_decode_kernel<512, 0, false, 4><<<grid, 256, 0, g->q>>>(p);
    } else {
        if (LW == 256) mla_decode_kernel<256, 0, false, 8><<<grid, 512, 0, g->q>>>(p);
        else if (q8) mla_decode_kernel<512, 0, true, 8><<<grid, 512, 0, g->q>>>(p);
        else if (R == 64) mla_decode_kernel<512, 64, false, 8><<<grid, 512, 0, g->q>>>(p);
        else mla_decode_kernel<512, 0, false, 8><<<grid, 512, 0, g->q>>>(p);
    }
    NS_LAUNCHED("mla_decode");
    if (ns_profile_mark(g, 1)) return -1;
    if (ns > 1) {
        if (LW == 256) {
            if (ot == 0) mla_merge_kernel<256, 0><<<dim3((unsigned) rows, 1), 256, 0, g->q>>>(scratch, (int) ns, u);
            else mla_merge_kernel<256, 1><<<dim3((unsigned) rows, 1), 256, 0, g->q>>>(scratch, (int) ns, u);
        } else {
            if (ot == 0) mla_merge_kernel<512, 0><<<dim3((unsigned) rows, 2), 256, 0, g->q>>>(scratch, (int) ns, u);
            else mla_merge_kernel<512, 1><<<dim3((unsigned) rows, 2), 256, 0, g->q>>>(scratch, (int) ns, u);
        }
        NS_LAUNCHED("mla_merge");
        return ns_profile_mark(g, 2);
    }
    return 0;
}

}  // namespace

extern "C" {

// A prompt's rows (T past 16) go through the same kernel a pass of rows after another on the queue: 16 rows x H heads
// already fill the kernel's row groups, and a pass's arithmetic (2 x rows H x cells x 1088 flop) outweighs its read of
// the cache, so nothing is gained by a second kernel. Every row of a pass walks the cells of the pass's last row (the
// later ones masked), so a pass is 128 rows (behind a short context the masked work is small in absolute terms and a
// pass costs its two launches), 256 = MLA_PASS_MAX once the masked part stays under a quarter. The scratch is
// the largest pass's.
// (17 to 27 row groups of 128 (row, head) pairs fill an XCD's 32 places once and little more: behind 4096 cells and more
// such a pass is cut at 16 groups - 17 rows x 128 heads behind 32768 cells: 274 us as one pass, 152 + 27 as two)
static int64_t mla_pass_rows(int64_t before, int64_t left, int64_t H) {
    int64_t w = 128;
    while (w < MLA_PASS_MAX && 8 * w <= before) w *= 2;
    const int64_t n = std::min(w, left), groups = (n * H + 127) / 128;
    return before >= 4096 && groups >= 17 && groups <= 27 && 16 * 128 / H >= 1 ? std::min<int64_t>(n, 16 * 128 / H) : n;
}
static int64_t mla_pass_scratch(int64_t T, int64_t H, int64_t pos0) {
    const int64_t rows = T * H, cells = pos0 + T, MROWS = mla_waves(rows, cells) * 16, nz = (rows + MROWS - 1) / MROWS, kbs = mla_kbs(cells, nz);
    return rows * ((cells + kbs - 1) / kbs) * PSTRIDE;
}

int64_t ns_mla_decode_latent_scratch(int64_t T, int64_t H, int64_t pos0) {
    if (T <= 0 || H <= 0) return 0;
    if (T <= 16) return mla_pass_scratch(T, H, pos0);
    int64_t need = 0;
    for (int64_t t0 = 0, n; t0 < T; t0 += n) {
        n = mla_pass_rows(pos0 + t0, T - t0, H);
        need = std::max(need, mla_pass_scratch(n, H, pos0 + t0));
    }
    return need;
}

int ns_mla_decode_latent(ns_gpu* g, int qt, const void* qa, const uint16_t* cache, void* u, int64_t T, int64_t H, int64_t R, int64_t pos0,
                         float scale, float* scratch) {
    NS_TRY
    if (T <= 0) return 0;
    if (qt != 0 && qt != 1) return ns_fail("ns_mla_decode_latent: rows of type 0 (float32) or 1 (half)");
    if (R != 0 && R != 64) return ns_fail("ns_mla_decode_latent: a rope part of 64 (DeepSeek's [512 | 64] rows) or none");
    if (H <= 0 || pos0 < 0) return ns_fail("ns_mla_decode_latent: heads and a position");
    if (!qa || !u) return ns_fail("ns_mla_decode_latent: a null buffer");
    const int64_t e = qt == 0 ? 4 : 2;
    for (int64_t t0 = 0, n; t0 < T; t0 += n) {
        n = T <= 16 ? T : mla_pass_rows(pos0 + t0, T - t0, H);
        if (mla_latent(g, "ns_mla_decode_latent", qt, qt, (int) R, false, (const char*) qa + t0 * H * (ML + R) * e, cache, (char*) u + t0 * H * ML * e, n, H,
                       pos0 + t0, scale, scratch, (size_t) mla_pass_scratch(n, H, pos0 + t0)))
            return -1;
    }
    return 0;
    NS_CATCH
}

// one body for both weight forms (kvb != NULL: Q6_K rows). More rows than a decode pass holds are queued 16 at a time - the
// reference's kernel takes any row count (kernels/llm/deepseek2/ds2.cpp:262-281), its engine sends prompts elsewhere
static int ds2_decode(ns_gpu* g, const char* who, const float* q, const uint16_t* kb, const uint16_t* vb, const uint8_t* kvb, const uint16_t* cache,
                      float* out, int64_t T, int64_t H, int64_t pos0, float scale) {
    const std::string w(who);
    if (T <= 0) return 0;
    if (H <= 0 || pos0 < 0) return ns_fail(w + ": heads and a position");
    if (!q || !cache || !out || (kvb ? false : !kb || !vb)) return ns_fail(w + ": a null buffer");
    if (kvb && (uintptr_t) kvb % 2) return ns_fail(w + ": kv_b 2-byte aligned");
    NS_HIP(hipSetDevice(g->dev));
    for (int64_t t0 = 0; t0 < T; t0 += 16) {
        const int64_t n = std::min<int64_t>(16, T - t0);
        // the library's own scratch (the reference's signature has none): the absorbed queries, u, then the partials
        const size_t rows = (size_t) (n * H), qa_f = (rows * (ML + 64) + 3) / 4 * 4, u_f = rows * ML;
        if (qa_f + u_f + rows * PSTRIDE > ns_own_floats(g)) return ns_fail(w + ": the pass needs more scratch than the library keeps");
        // (the absorbed queries as halfs - the rounding the latent kernel gives float32 rows on their way into its first
        // product - so its work-groups fetch half the bytes before their first tile: 24.4 -> 21 us of the kernel at one row)
        uint16_t* qa = reinterpret_cast<uint16_t*>(g->own_scratch);
        float* u = g->own_scratch + qa_f;
        float* part = u + u_f;
        const float* qp = q + t0 * H * 192;
        float* op = out + t0 * H * 128;
        if (kvb) mla_absorb_q6k_kernel<<<(unsigned) rows, 256, 0, g->q>>>(qp, kvb, qa, H);
        else mla_absorb_kernel<<<dim3((unsigned) rows, 4), 256, 0, g->q>>>(qp, kb, qa, H);
        NS_LAUNCHED("mla_absorb");
        if (mla_latent(g, who, 1, 0, 64, false, qa, cache, u, n, H, pos0 + t0, scale, part, ns_own_floats(g) - qa_f - u_f)) return -1;
        if (kvb) mla_vb_q6k_kernel<<<dim3((unsigned) rows, 4), 256, 0, g->q>>>(u, kvb, op, H);
        else mla_vb_kernel<<<dim3((unsigned) rows, 4), 256, 0, g->q>>>(u, vb, op, H);
        NS_LAUNCHED("mla_vb");
    }
    return 0;
}

int ns_ds2_mla_decode(ns_gpu* g, const float* q, const uint16_t* kb, const uint16_t* vb, const uint16_t* cache, float* out, int64_t T, int64_t H,
                      int64_t pos0, float scale) {
    NS_TRY
    return ds2_decode(g, "ns_ds2_mla_decode", q, kb, vb, nullptr, cache, out, T, H, pos0, scale);
    NS_CATCH
}

int ns_ds2_mla_decode_q6k(ns_gpu* g, const float* q, const void* kvb, const uint16_t* cache, float* out, int64_t T, int64_t H, int64_t pos0,
                          float scale) {
    NS_TRY
    if (T > 0 && !kvb) return ns_fail("ns_ds2_mla_decode_q6k: a null buffer");
    return ds2_decode(g, "ns_ds2_mla_decode_q6k", q, nullptr, nullptr, (const uint8_t*) kvb, cache, out, T, H, pos0, scale);
    NS_CATCH
}

int ns_ds2_rope(ns_gpu* g, float* x, int64_t T, int64_t H, int64_t row, int64_t head, int64_t off, int64_t n_dims, int64_t pos0,
                float freq_base, float freq_scale, float ext_factor, float mscale, float corr0, float corr1, float* out, int64_t out_row,
                int64_t out_head) {
    NS_TRY
    if (n_dims % 2 != 0) return ns_fail("ns_ds2_rope: an even rotated width");
    if (T <= 0 || H <= 0 || n_dims <= 0) return 0;
    if (!g || !x) return ns_fail("ns_ds2_rope: a null buffer");
    NS_HIP(hipSetDevice(g->dev));
    ds2_rope_kernel<<<(unsigned) ((T * H * (n_dims / 2) + 255) / 256), 256, 0, g->q>>>(x, T, H, row, head, off, n_dims, pos0, freq_base, freq_scale, ext_factor,
                                                                            mscale, corr0, corr1, out, out_row, out_head);
    NS_LAUNCHED("ds2_rope");
    return 0;
    NS_CATCH
}

int ns_ds2_kv_store(ns_gpu* g, const float* kv, const float* w, float eps, uint16_t* cache, int64_t T, int64_t L, int64_t R, int64_t pos0,
                    float freq_base, float freq_scale, float ext_factor, float mscale, float corr0, float corr1) {
    NS_TRY
    if (T <= 0) return 0;
    if (L <= 0 || R < 0 || R % 2 != 0 || pos0 < 0) return ns_fail("ns_ds2_kv_store: a latent width, an even rotated width and a position");
    if (!g || !kv || !w || !cache) return ns_fail("ns_ds2_kv_store: a null buffer");
    NS_HIP(hipSetDevice(g->dev));
    ds2_kv_store_kernel<<<(unsigned) T, 256, 0, g->q>>>(kv, w, eps, cache, L, R, pos0, freq_base, freq_scale, ext_factor, mscale, corr0, corr1);
    NS_LAUNCHED("ds2_kv_store");
    return 0;
    NS_CATCH
}

// GLM's latent-only MLA through the library's own scratch, any number of rows: rows with cell lists of their own go 16 a
// pass (a row group holds one row's heads, so wider passes gain nothing), dense rows as a prompt's do
static int mla_sel_rows(ns_gpu* g, const char* who, bool q8, const float* qa, const void* c, float* u, int64_t T, int64_t H, int64_t pos0,
                        float scale, const int32_t* sel, const int32_t* sel_cnt, int64_t K, float* scratch, size_t scratch_floats, int LW = 512) {
    if (H <= 0 || pos0 < 0) return ns_fail(std::string(who) + ": heads and a position");
    if (!qa || !u) return ns_fail(std::string(who) + ": a null buffer");
    for (int64_t t0 = 0, n; t0 < T; t0 += n) {
        n = T <= 16 ? T : sel_cnt ? std::min<int64_t>(16, T - t0) : mla_pass_rows(pos0 + t0, T - t0, H);
        if (mla_latent(g, who, 0, 0, 0, q8, qa + t0 * H * LW, c, u + t0 * H * LW, n, H, pos0 + t0, scale, scratch, scratch_floats,
                       sel_cnt ? sel + t0 * K : nullptr, sel_cnt ? sel_cnt + t0 : nullptr, K, LW))
            return -1;
    }
    return 0;
}

int ns_mla_attend_sel(ns_gpu* g, const float* qa, const uint16_t* c, float* u, int64_t T, int64_t H, int64_t L, int64_t pos0, float scale,
                      const int32_t* sel, const int32_t* sel_cnt, int64_t K) {
    NS_TRY
    if (T <= 0) return 0;
    // (both of the reference's widths, kernels/llm/glm5next/glm.cpp:1254-1266, each an instance of the latent kernel)
    if (L != 256 && L != 512) return ns_fail("ns_mla_attend_sel: latent width 256 or 512");
    return mla_sel_rows(g, "ns_mla_attend_sel", false, qa, c, u, T, H, pos0, scale, sel, sel_cnt, K, g->own_scratch, ns_own_floats(g), (int) L);
    NS_CATCH
}

int ns_mla_attend_sel_q8(ns_gpu* g, const float* qa, const void* c, float* u, int64_t T, int64_t H, int64_t L, int64_t pos0, float scale,
                         const int32_t* sel, const int32_t* sel_cnt, int64_t K) {
    NS_TRY
    if (T <= 0) return 0;
    if (L != 512) return ns_fail("ns_mla_attend_sel_q8: latent width 512");
    return mla_sel_rows(g, "ns_mla_attend_sel_q8", true, qa, c, u, T, H, pos0, scale, sel, sel_cnt, K, g->own_scratch, ns_own_floats(g));
    NS_CATCH
}

// the dense form over a float32 latent cache c [n][512]: its rows 0 .. pos0 + T - 1 are rounded to half into the
// library's scratch (the half cache's own rounding) and the latent kernel reads those
int ns_mla_attend(ns_gpu* g, const float* qa, const float* c, float* u, int64_t T, int64_t H, int64_t L, int64_t pos0, float scale) {
    NS_TRY
    if (T <= 0) return 0;
    if (L != 256 && L != 512) return ns_fail("ns_mla_attend: latent width 256 or 512");
    if (pos0 < 0 || !c) return ns_fail("ns_mla_attend: a position and a cache");
    if ((uintptr_t) c % 16) return ns_fail("ns_mla_attend: the cache 16-byte aligned");
    const int64_t cells = pos0 + T, ch_floats = (cells * L / 2 + 3) / 4 * 4;      // the half rows, counted in floats
    if ((size_t) ch_floats + (size_t) (H > 0 ? 16 * H * PSTRIDE : 0) > ns_own_floats(g))
        return ns_fail("ns_mla_attend: more cells than the library's scratch holds as half rows (use a half cache and ns_mla_attend_sel)");
    NS_HIP(hipSetDevice(g->dev));
    uint16_t* ch = (uint16_t*) g->own_scratch;
    to_half_kernel<<<(unsigned) ((cells * L / 8 + 255) / 256), 256, 0, g->q>>>(c, ch, cells * L / 8);
    NS_LAUNCHED("to_half");
    return mla_sel_rows(g, "ns_mla_attend", false, qa, ch, u, T, H, pos0, scale, nullptr, nullptr, 0, g->own_scratch + ch_floats,
                        ns_own_floats(g) - (size_t) ch_floats, (int) L);
    NS_CATCH
}

int ns_gather_q8_h(ns_gpu* g, const void* src, const int32_t* idx, uint16_t* out, int64_t n, int64_t L) {
    NS_TRY
    if (n <= 0) return 0;
    if (L != 512) return ns_fail("ns_gather_q8_h: latent width 512");
    if (!src || !idx || !out) return ns_fail("ns_gather_q8_h: a null buffer");
    if ((uintptr_t) src % 8 || (uintptr_t) out % 16) return ns_fail("ns_gather_q8_h: rows 8-byte, the output 16-byte aligned");
    NS_HIP(hipSetDevice(g->dev));
    gather_q8_h_kernel<<<(unsigned) ((n * 64 + 255) / 256), 256, 0, g->q>>>((const uint8_t*) src, idx, out, n);
    NS_LAUNCHED("gather_q8_h");
    return 0;
    NS_CATCH
}

int ns_to_q8row(ns_gpu* g, const float* x, void* y, int64_t n, int64_t L) {
    NS_TRY
    if (n <= 0) return 0;
    if (L != 512) return ns_fail("ns_to_q8row: latent width 512");
    if (!g || !x || !y) return ns_fail("ns_to_q8row: a null buffer");
    if ((uintptr_t) x % 16 || (uintptr_t) y % 4) return ns_fail("ns_to_q8row: float rows 16-byte, q8 rows 4-byte aligned");
    NS_HIP(hipSetDevice(g->dev));
    to_q8row_kernel<<<(unsigned) ((n * 16 + 255) / 256), 256, 0, g->q>>>(x, (uint8_t*) y, n);
    NS_LAUNCHED("to_q8row");
    return 0;
    NS_CATCH
}

}  // extern "C"
