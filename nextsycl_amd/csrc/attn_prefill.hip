// attn_prefill.hip: causal GQA flash attention of a prompt pass's rows against the KV cache (half, bfloat16, q8_0 or q4_0
// rows; D = 128 or 256) for gfx950.
//
// Bound: MFMA. 4 D flops a visible (row, key) pair against 2 x 2 D bytes a key shared by every row that sees it:
// thousands of flops a byte at prompt lengths.
//
// Work split: one work-group per (row block, query head). A work-group of 8 waves owns ROWS = 256 consecutive query rows
// of one query head (a wave 32 of them: two 16-row MFMA tiles) and streams the keys its rows see in 64-key tiles,
// heaviest row blocks first (the last block sees the most keys). The G query heads of a key head on one row block are
// neighbours in the logical order and, through the XCD-aware mapping of work-group ids, share one L2. A tile's K and V
// rows are fetched by all the work-group's threads (16-byte chunks). Over 16-bit rows at D = 128 they go global -> LDS
// directly (global_load_lds_dwordx4, unpadded buffers, the bank swizzle applied to the global addresses, one barrier a
// tile that waits on the wave's transfers): the 8-wave form two tiles ahead into three buffers a stream, the barrier
// leaving the newest tile's transfers in flight; the 4-wave form (two work-groups a CU) one tile ahead into two buffers a
// stream, requested right behind the barrier that frees them. The other forms (quantized rows, D = 256) go global ->
// registers two tiles ahead -> LDS one tile ahead: two register sets, two padded LDS buffers.
// A pass of few rows packs several query heads of one key head into a work-group (a wave slot a head: the tile staged
// once serves them all), and a pass of few rows over a long context is cut into key splits whose partials a merge
// kernel puts together. bfloat16, q8_0 and q4_0 rows read many times are first widened to half rows in the library's
// scratch (bit for bit the halfs the kernel would stage); the kernel's own forms of them serve short passes and caches
// the scratch does not hold.
//
// A wave's tile step, in the transposed orientation (a lane owns one query row of each row tile, so the row maximum,
// the rescale and the normalisation never leave the lane):
//   S^T[key][row] = K Q^T        K from LDS as the A operand (ds_read_b128; rows padded to 288 bytes, or swizzled), Q^T in registers.
//                                Half operands: Q carries the softmax scale x log2 e and the product starts from minus the
//                                softmax reference, so a score leaves the matrix unit as the argument of its exponential
//   base-2 online softmax in float32 (the accumulators rescaled only when a row's maximum moved); only 32-key halves
//   crossing a row's causal or window edge are masked
//   P^T -> 16 bit = the B operand of the second product as it stands
//   O^T[d][row]  += V^T P^T      V^T from LDS through ds_read_b64_tr_b16 (rows padded to 288 bytes, or swizzled)
//
// Reference behaviour kept: kernels/llm/museglimmer/silo/attn.cpp:56-267 and kernels/llm/qwen35/silo/attn.cpp:105-313
// (prompt form: causal from p0, window, ring slots, 16-bit operands with float32 softmax and accumulation, rows past T
// not written, no scratch).
#include "ns_internal.hpp"
#include "ns_attn.h"
#include "attn_common.hpp"
#include "attn_host.hpp"
#include "kv_formats.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <type_traits>


namespace {

constexpr int KT_TILE = 64;
// waves a work-group (PW): at D = 128 a wave owns 32 rows and a work-group 8 waves = 256 rows when that still leaves two
// work-groups for every CU - a tile staged for 256 rows costs half the fetches and LDS writes a row, and two work-groups
// of 4 waves on a CU were measured to run no faster than one of 8 - else 4 waves = 128 rows; at D = 256 4 waves of 16 rows
constexpr int rows_of(int D, int PW) { return PW * (D == 128 ? 32 : 16); }   // query rows a work-group

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
    int causal;                 // 0: every row sees to the pass's last key (a draft block)
    int64_t kfirst;             // >= 0: every row's first key, instead of its own window's
    float sl2;
    void* out;
    // key splits (passes of few row blocks over many keys): work-group (x, y) takes the keys [k0 + y kbs, k0 + (y + 1) kbs)
    // of its rows' own ranges and leaves a partial {O, m, l} a (row, head, split) for the decode path's merge kernel
    int ns;
    int64_t kbs, k0;
    float* part;                // [T][Hq][ns][D + 2]
    // a pass of few rows: a work-group holds `pack` query heads of its key head - wave w rows (w / pack) x (a wave's rows)
    // .. of head w % pack - so the heads share every key and value tile the work-group stages. 1: one head, every wave rows
    // of its own. gw = G / pack: work-groups a (row block, key head)
    int pack, gw;
};

// a 16-byte chunk of a K or V row on its way from global memory to LDS (a plain vector type: arrays of it stay in registers)
typedef uint32_t u4v __attribute__((ext_vector_type(4)));
// the same at an address that is only 8-byte aligned (q8_0 / q4_0 rows of 128 values are 136 / 72 bytes long)
typedef uint32_t u4a8 __attribute__((ext_vector_type(4), aligned(8)));

// BF: bfloat16 operands (a bfloat16 cache too long to be widened to half first), else half. QS (bfloat16 operands only):
// query rows of another type enter the first product as two bfloat16 numbers - the rounded row and the rounded rest, 16
// significant bits between them - a second matrix instruction a key block.
// NTS (16-bit rows of 128 only): the tiles' transfers carry the streaming cache policy - a pass whose keys are each read
// by one work-group, once.
template <int D, bool BF, int KT, int PW, bool QS = false, bool NTS = false>
__global__ __launch_bounds__(PW * 64, PW == 4 && D == 128 ? 2 : 1) void attn_prefill_kernel(const PrefillParams p) {
    static_assert(D == 128 || D == 256, "head size 128 or 256");
    static_assert(KT == 0 || !BF, "quantized rows are widened to half");
    static_assert(!QS || BF, "query rows in two parts: bfloat16 operands only");
    // a wave owns RT row tiles of 16: 32 rows at D = 128; 16 at D = 256, whose accumulators are twice as wide
    constexpr int RT = D == 128 ? 2 : 1, WROWS = RT * 16;
    constexpr int KB = D / 32, DT = D / 16;
    // Half operands: the query enters the first product scaled by the softmax scale x log2 e and rounded once to half - what
    // the reference's kernels do (qwen35/silo/attn.cpp:112,147: qh = half(q x qscale)) - and the product starts from minus
    // the softmax reference (ntile), so a score leaves the matrix unit as the argument of its exponential: no vector
    // instruction a score between the two. bfloat16 operands (8 bits: a second rounding would show) keep the scale in a
    // fused multiply-add a score.
    constexpr bool PRESCALE = !BF;
    // bytes a staged key row / value row: rows 32 bytes apart modulo 256, so that the 16-byte operand reads of 16 keys (and
    // the transposing reads of the values) meet no bank conflict - 16 bytes apart the key reads would, two ways
    constexpr int KS = D * 2 + 32, VS = D * 2 + 32;
    constexpr int KBUF = KT_TILE * KS, VBUF = KT_TILE * VS;
    // DMA: 8 waves over 16-bit rows of 128 stage their tiles global -> LDS directly (global_load_lds_dwordx4: no register in
    // between, no LDS write instruction, a tile requested two tiles ahead). The tiles are unpadded 256-byte rows, a row's
    // 16-byte chunks exclusive-ored into place by its key (keys: chunk c of key r at position c ^ (r % 16); values:
    // c ^ 2 (r % 8)) so that neither the operand reads of 16 keys' same chunk nor the transposing reads meet a bank
    // conflict; three buffers a stream, each an array of its own so that the compiler can tell a transfer's target from
    // the arrays being read (it waits for every transfer in flight before a read it cannot tell apart)
    // The 4-wave form (two work-groups a CU) has LDS for two buffers a stream: a tile is then requested one tile ahead,
    // right behind the barrier that frees its buffer, and the next barrier waits for every transfer of the wave.
    constexpr bool DMA = D == 128 && KT == 0 && (PW == 8 || PW == 4);
    constexpr int NBUF = PW == 8 ? 3 : 2;                         // tile buffers a stream
    constexpr int NJ = 16 / PW;                                   // transfer instructions a wave, tile and stream
    constexpr int TB = KT_TILE * 256;
    constexpr int TBP = TB + 512;                                 // (two waves' output staging, 8448 B each, go through one array)
    __shared__ __attribute__((aligned(16))) uint8_t lds[DMA ? 16 : 2 * (KBUF + VBUF)];
    __shared__ __attribute__((aligned(1024))) uint8_t dk0[DMA ? TBP : 16];
    __shared__ __attribute__((aligned(1024))) uint8_t dk1[DMA ? TBP : 16];
    __shared__ __attribute__((aligned(1024))) uint8_t dk2[DMA && NBUF == 3 ? TBP : 16];
    __shared__ __attribute__((aligned(1024))) uint8_t dv0[DMA ? TBP : 16];
    __shared__ __attribute__((aligned(1024))) uint8_t dv1[DMA ? TBP : 16];
    __shared__ __attribute__((aligned(1024))) uint8_t dv2[DMA && NBUF == 3 ? TBP : 16];

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 15, g4 = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    // ---- which (row block, head) this work-group owns. Consecutive work-group ids go round the 8 XCDs (each with its
    // own L2). The G query heads of one key head on one row block stream the same K / V tiles: they are one unit, and a
    // unit's work-groups are consecutive on one XCD. Units are dealt to the XCDs round-robin in order of weight (the last
    // row block sees the most keys), so every XCD gets the same mix of heavy and light units, heaviest first. The grid is
    // padded to a multiple of 8 units; the work-groups of the padding leave at once.
    const int pid = blockIdx.x, xcd = pid % 8, xi = pid / 8;
    const int pk = p.pack, wh = w % pk, wr = w / pk;              // (scalars: this wave's head of the work-group's, its rows' place)
    const int wslots = PW / pk;                                   // waves a head (a wave past pk x wslots has no rows: 5 heads to 8 waves)
    const int RB = wslots * WROWS;                                // rows of a head a work-group holds
    const int nblk = (p.T + RB - 1) / RB;
    const int Hkv = p.Hq / p.G;
    // (with key splits a split is one more factor of the units, the slowest: a pass of fewer than 8 units still puts work on
    // every XCD, and a unit's splits - different keys - go to different ones)
    const int nun = nblk * Hkv, u2 = (xi / p.gw) * 8 + xcd;
    if (u2 >= nun * p.ns) return;
    const int unit = u2 % nun;
    const int hk = unit % Hkv;
    const int hq = hk * p.G + (xi % p.gw) * pk + wh;
    const int blk = nblk - 1 - unit / Hkv;
    const int r0 = blk * RB;
    const int rl = std::min(r0 + RB, p.T) - 1;                    // the block's last row
    const int wbase = wr < wslots ? r0 + wr * WROWS : p.T;        // this wave's first row (none: past the pass's last)
    // keys [kbeg, kend) cover every row of the block; with key splits, the part of them in this work-group's split
    const int split = u2 / nun;
    int64_t kend = p.causal ? p.p0 + rl + 1 : p.p0 + p.T;
    int64_t kbeg = p.kfirst >= 0 ? p.kfirst : p.win > 0 ? std::max<int64_t>(0, p.p0 + r0 + 1 - p.win) : 0;
    if (p.ns > 1) {
        kbeg = std::max(kbeg, p.k0 + split * p.kbs);
        kend = std::max(kbeg, std::min(kend, p.k0 + (split + 1) * p.kbs));      // (none: an empty range at kbeg)
    }

    // ---- this lane's two rows: positions, key ranges, Q^T operands
    int64_t lo_r[RT], hi_r[RT];
    s8v qreg[RT][KB], qlo[QS ? RT : 1][KB];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int row = wbase + rt * 16 + n;
        const bool live = row < p.T;
        const int rr = live ? row : p.T - 1;
        const int64_t pos = p.p0 + rr;
        lo_r[rt] = live ? std::max(kbeg, p.kfirst >= 0 ? p.kfirst : p.win > 0 ? std::max<int64_t>(0, pos + 1 - p.win) : 0) : 1;
        hi_r[rt] = live ? std::min(p.causal ? pos : p.p0 + p.T - 1, kend - 1) : 0;
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
                for (int i = 0; i < 8; ++i) {
                    qreg[rt][kb][i] = to16<BF>(PRESCALE ? f[i] * p.sl2 : f[i]);
                    if constexpr (QS) qlo[rt][kb][i] = to16<true>(f[i] - bf16_to_f32((uint16_t) qreg[rt][kb][i]));
                }
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
                    // bfloat16 operands: rows of that type pass through bit for bit, others are rounded once; half operands:
                    // the row x the scale, rounded once
                    if constexpr (PRESCALE) qreg[rt][kb][i] = to16<BF>((p.qt == 1 ? f16_to_f32(b16) : bf16_to_f32(b16)) * p.sl2);
                    else qreg[rt][kb][i] = (p.qt == 2) == BF ? (short) b16 : to16<BF>(p.qt == 1 ? f16_to_f32(b16) : bf16_to_f32(b16));
                    if constexpr (QS) qlo[rt][kb][i] = p.qt == 1 ? to16<true>(f16_to_f32(b16) - bf16_to_f32((uint16_t) qreg[rt][kb][i])) : (short) 0;
                }
            }
        }
    }
    const uint8_t* kbase = p.kc + (int64_t) hk * p.head_stride;
    const uint8_t* vbase = p.vc + (int64_t) hk * p.head_stride;
    const int64_t t0 = kbeg / KT_TILE, t1 = (kend + KT_TILE - 1) / KT_TILE;
    const int nt = kend > kbeg ? (int) (t1 - t0) : 0;             // (a split past the block's last key: nothing to do)
    // From here on keys are counted from the first tile's first key (32-bit): tile k holds keys 64 k .. 64 k + 63, step
    // s = 2 k + h its 32-key half h
    const int64_t base = t0 * KT_TILE;
    int lo32[RT], hi32[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const bool live = wbase + rt * 16 + n < p.T;
        lo32[rt] = live ? (int) (lo_r[rt] - base) : 1;
        hi32[rt] = live ? (int) (hi_r[rt] - base) : 0;
    }
    // the wave's own steps: from its first row's first key to its last row's last; steps in between that no row's edge
    // crosses need no mask
    const int wrow0 = wbase, wrow1 = std::min(wrow0 + WROWS - 1, p.T - 1);
    const int w_full_end = (int) ((p.causal ? p.p0 + wrow0 + 1 : p.p0 + p.T) - base);
    const int w_full_beg = p.kfirst >= 0 ? (int) (p.kfirst - base) : p.win > 0 ? (int) (std::max<int64_t>(0, p.p0 + wrow1 + 1 - p.win) - base) : 0;

    // Online softmax state, in base-2 exponent units (scores x scale x log2 e): nbr = minus the reference the weights
    // are taken against, thr = how far a score may exceed it before the reference moves (-inf while the row has seen no
    // key: the first one sets it). The row's sum of weights l4 comes out of the matrix unit: a product of the rounded weights
    // with an operand of ones beside each step's V^T P^T (every slot of l4 then holds the whole row's sum - no vector
    // additions, no cross-lane step, and numerator and denominator carry the very same rounded weights)
    float nbr[RT], thr[RT];
    f4v l4[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        nbr[rt] = 0.0f;
        thr[rt] = -INFINITY;
        l4[rt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
    }
    f4v o[RT][DT], ntile[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        ntile[rt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[rt][dt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
    }

    // ---- global -> registers -> LDS. A cache row is fetched in 16-byte raw chunks: 16-bit rows D / 8 of them, each one
    // LDS piece; q8_0 rows D / 16 (16 int8 -> 2 pieces of 8 halfs, the block's half scale fetched beside it); q4_0 rows
    // D / 32 (one block: 32 nibbles -> 4 pieces). A thread's chunks of a tile: chunk c = tid + 256 i -> key c / CPR, raw
    // chunk c % CPR. A tile wholly inside [kbeg, kend) of an unwrapped cache is read at a wave-uniform address plus a
    // 32-bit lane offset; otherwise keys outside are clamped into the range (a valid row, masked; a tile past the last
    // is fetched as the last row over and over and never used) and a wrapped ring's slot is position % cap: the first
    // key's once, then offsets from it with at most two wraps (a pass's keys span less than two rings)
    constexpr int CPR = KT == 0 ? D / 8 : KT == 1 ? D / 16 : D / 32;             // raw chunks a row
    constexpr int NST = KT_TILE * CPR / (PW * 64);                                // raw chunks a thread per tile
    constexpr int KPI = PW * 64 / CPR;                                            // keys between a thread's chunks
    constexpr int PPC = KT == 0 ? 1 : KT == 1 ? 2 : 4;                            // LDS pieces a raw chunk
    static_assert(NST >= 1 && NST * PW * 64 == KT_TILE * CPR, "whole chunks a thread");
    struct Stage {
        u4v raw[NST];
        uint16_t sc[KT == 0 ? 1 : NST];
    };
    const int64_t kbeg_slot = p.wrap ? kbeg % p.cap : kbeg;
    const int kspan = (int) (kend - kbeg) - 1;
    const int kbeg32 = (int) (kbeg - base);
    const int key0 = tid / CPR, rc = tid % CPR;                   // chunk i of this thread: key key0 + KPI i, raw chunk rc
    const uint32_t lane_off = (uint32_t) (key0 * p.row_stride) + (uint32_t) rc * 16;
    // where a chunk's scale sits in its row: q8_0 a half a block of 32 behind D values, q4_0 behind D / 2 bytes
    // (as a distance from the chunk itself)
    const uint32_t sc_rel = (KT == 1 ? (uint32_t) (D + 2 * (rc / 2)) : (uint32_t) (D / 2 + 2 * rc)) - (uint32_t) rc * 16;
    const int plain0 = kbeg32 > 0 ? 1 : 0, plain1 = p.wrap ? -1 : (int) ((kend - base) / KT_TILE) - 1;
    auto fetch = [&](Stage& st, const uint8_t* cache, int krel) {
        const int64_t rs = p.row_stride;
        const bool wrap = p.wrap;
        const uint8_t* sp = cache;
        uint32_t off[NST];                                        // of the raw chunk
        if (krel >= plain0 && krel <= plain1) {
            sp += (base + (int64_t) krel * KT_TILE) * rs;
#pragma unroll
            for (int i = 0; i < NST; ++i) off[i] = lane_off + (uint32_t) (i * KPI * rs);
        } else {
            const int rel0 = krel * KT_TILE - kbeg32 + key0;
#pragma unroll
            for (int i = 0; i < NST; ++i) {
                const int rel = std::min(std::max(rel0 + KPI * i, 0), kspan);
                int64_t slot = kbeg_slot + rel;
                if (wrap) {
                    slot = slot >= p.cap ? slot - p.cap : slot;
                    slot = slot >= p.cap ? slot - p.cap : slot;
                }
                off[i] = (uint32_t) (slot * rs) + (uint32_t) rc * 16;   // a head's cache spans less than 4 GiB
            }
        }
#pragma unroll
        for (int i = 0; i < NST; ++i) {
            if constexpr (KT != 0 && D == 128) st.raw[i] = *reinterpret_cast<const u4a8*>(sp + off[i]);
            else st.raw[i] = *reinterpret_cast<const u4v*>(sp + off[i]);
            if constexpr (KT != 0) st.sc[i] = *reinterpret_cast<const uint16_t*>(sp + off[i] + sc_rel);
        }
    };
    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    lds_u8* const L = (lds_u8*) lds;
    // LDS map: K tiles at 0 and KBUF, V tiles at 2 KBUF and 2 KBUF + VBUF; rows of D halfs (+ padding) whatever the cache
    constexpr uint32_t V0 = 2 * KBUF;
    // a raw chunk's pieces written at row stride RS from byte offset at (quantized rows widened: one rounding to half of
    // (float) q x (float) scale, what the reference stages - qwen35/silo/attn.cpp:56-76)
    const uint32_t k_wr = (uint32_t) (key0 * KS + rc * 16 * PPC), v_wr = (uint32_t) (key0 * VS + rc * 16 * PPC);
    auto put = [&](const Stage& st, uint32_t at0, int RS) {
#pragma unroll
        for (int i = 0; i < NST; ++i) {
            const uint32_t at = at0 + (uint32_t) (i * KPI * RS);
            if constexpr (KT == 0) {
                *reinterpret_cast<__attribute__((address_space(3))) u4v*>(L + at) = st.raw[i];
            } else {
                const _Float16 d = __builtin_bit_cast(_Float16, st.sc[i]);
                if constexpr (KT == 1) {
                    *reinterpret_cast<__attribute__((address_space(3))) s8v*>(L + at) = dq8x8(st.raw[i][0], st.raw[i][1], d);
                    *reinterpret_cast<__attribute__((address_space(3))) s8v*>(L + at + 16) = dq8x8(st.raw[i][2], st.raw[i][3], d);
                } else {
                    // values 0 .. 15: the low nibbles of the 16 bytes, 16 .. 31: the high ones
                    *reinterpret_cast<__attribute__((address_space(3))) s8v*>(L + at) = dq4x8(st.raw[i][0], st.raw[i][1], 0, d);
                    *reinterpret_cast<__attribute__((address_space(3))) s8v*>(L + at + 16) = dq4x8(st.raw[i][2], st.raw[i][3], 0, d);
                    *reinterpret_cast<__attribute__((address_space(3))) s8v*>(L + at + 32) = dq4x8(st.raw[i][0], st.raw[i][1], 4, d);
                    *reinterpret_cast<__attribute__((address_space(3))) s8v*>(L + at + 48) = dq4x8(st.raw[i][2], st.raw[i][3], 4, d);
                }
            }
        }
    };
    auto stash_k = [&](const Stage& st, int buf) { put(st, (uint32_t) (buf * KBUF) + k_wr, KS); };
    auto stash_v = [&](const Stage& st, int buf) { put(st, V0 + (uint32_t) (buf * VBUF) + v_wr, VS); };

    // DMA: a wave's two 1 KiB instructions a tile and stream: instruction j fills rows 4 (2 w + j) .. + 3 of the tile (16
    // lanes a row: lane l position l % 16 of row 4 (2 w + j) + l / 16), so it fetches the chunk that belongs there. Whole
    // tiles of an unwrapped cache: a wave-uniform tile address plus lane offsets worked out once; else the row is clamped
    // into the pass's keys (masked anyway) and a ring's slot worked out, as the register path does
    uint32_t koff[DMA ? NJ : 1], voff[DMA ? NJ : 1];
    if constexpr (DMA) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int r = (w * NJ + j) * 4 + (lane >> 4), cp = lane & 15;
            koff[j] = (uint32_t) (r * p.row_stride) + (uint32_t) ((cp ^ (r & 15)) << 4);
            voff[j] = (uint32_t) (r * p.row_stride) + (uint32_t) ((cp ^ (2 * (r & 7))) << 4);
        }
    }
    // (one transfer instruction: 64 lanes x 16 bytes from base + the lane's offset to 1 KiB of LDS at dst, wave-uniform.
    // Written out so that the compiler's wait-count pass does not see a memory instruction that writes LDS - it would
    // make every later LDS read wait for all earlier ones; the waits these transfers need are the tile barrier's)
    auto dma16 = [&](const uint8_t* base_, uint32_t off, lds_u8* dst) __attribute__((always_inline)) {
        const uint32_t m = __builtin_amdgcn_readfirstlane((uint32_t) (uintptr_t) dst);
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"                   // (m0 is reserved: nothing of the compiler's lives in it across this)
        if constexpr (NTS) asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(m), "v"(off), "s"(base_) : "memory", "m0");
        else asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m), "v"(off), "s"(base_) : "memory", "m0");
#pragma clang diagnostic pop
    };
    auto dma = [&](lds_u8* dst, const uint8_t* cache, int krel, auto which_c) __attribute__((always_inline)) {
        constexpr bool VAL = decltype(which_c)::value;
        const int64_t rs = p.row_stride;
        const bool wrap = p.wrap;
        if (krel >= plain0 && krel <= plain1) {
            const uint8_t* sp = cache + (base + (int64_t) krel * KT_TILE) * rs;
#pragma unroll
            for (int j = 0; j < NJ; ++j)
                dma16(sp, VAL ? voff[j] : koff[j], dst + (w * NJ + j) * 1024);
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int r = (w * NJ + j) * 4 + (lane >> 4), cp = lane & 15;
                const int rel = std::min(std::max(krel * KT_TILE - kbeg32 + r, 0), kspan);
                int64_t slot = kbeg_slot + rel;
                if (wrap) {
                    slot = slot >= p.cap ? slot - p.cap : slot;
                    slot = slot >= p.cap ? slot - p.cap : slot;
                }
                const uint32_t off = (uint32_t) (slot * rs) + (uint32_t) ((VAL ? cp ^ (2 * (r & 7)) : cp ^ (r & 15)) << 4);
                dma16(cache, off, dst + (w * NJ + j) * 1024);
            }
        }
    };
    // a tile's barrier. DMA: this wave's transfers of the tile about to be read are done when at most the two younger
    // requests (2 instructions each) are still in flight, and every LDS read it has issued has returned (a wave past the
    // barrier may request a transfer into a buffer this wave read from); a bare barrier then - no fence over the
    // transfers still in flight
    auto tile_barrier = [&]() __attribute__((always_inline)) {
        if constexpr (DMA) {
            if constexpr (NBUF == 3) asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        } else {
            __syncthreads();
        }
    };
    const uint32_t k_rd = (uint32_t) (n * KS + g4 * 16);                          // + kt2 * 16 * KS + kb * 64
    const uint32_t v_rd = (uint32_t) ((g4 * 4 + (n >> 2)) * VS + (n & 3) * 8);    // + dt * 32 (+ 16 * VS)
    // (DMA tiles: where the lane's key-operand chunk kb and value-operand column tile dt sit in their swizzled rows)
    uint32_t k_rd4[DMA ? KB : 1], v_rd8[DMA ? DT : 1];
    if constexpr (DMA) {
        const int kkv = g4 * 4 + (n >> 2);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) k_rd4[kb] = (uint32_t) (n * 256 + (((kb * 4 + g4) ^ n) << 4));
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) v_rd8[dt] = (uint32_t) (kkv * 256 + ((dt ^ (kkv & 7)) << 5) + (((n & 3) >> 1) << 4) + (n & 1) * 8);
    }
    // (bfloat16 operands: a weight enters the second product as two bfloat16 numbers, the rounded weight pb and the rounded
    // rest pl - 16 significant bits between them, where one alone would carry 8 and cost the output ~1.6e-3 of relative L2)
    s8v pb[RT], pl[BF ? RT : 1];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) pb[rt] = s8v{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int rt = 0; rt < (BF ? RT : 1); ++rt) pl[rt] = s8v{0, 0, 0, 0, 0, 0, 0, 0};
    // S^T of one 32-key half (LDS byte offset kl) against the wave's 32 rows: the raw dot products
    // (the operands of a block's first matrix instructions are read a block earlier - kread / vread - so that their LDS
    // latency passes under the other block's work instead of at the head of this one)
    // (rows in two parts: the registers of half the value operands read ahead go to the rows' second part - no spills)
    constexpr int VPRE = D == 128 && !QS ? DT : 4;                // value operands read ahead
    constexpr int KPRE = D == 128 ? 2 : 1;                        // 16-key halves whose key operands are read ahead
    auto kread = [&](s8v (&ka)[KPRE][KB], const lds_u8* kl) __attribute__((always_inline)) {
#pragma unroll
        for (int kt2 = 0; kt2 < KPRE; ++kt2)
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                if constexpr (DMA) ka[kt2][kb] = *reinterpret_cast<const __attribute__((address_space(3))) s8v*>(kl + k_rd4[kb] + kt2 * 16 * 256);
                else ka[kt2][kb] = *reinterpret_cast<const __attribute__((address_space(3))) s8v*>(kl + k_rd + kt2 * 16 * KS + kb * 64);
            }
    };
    auto vread1 = [&](const lds_u8* vl, int dt) __attribute__((always_inline)) {
        if constexpr (DMA) {
            const s4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*) (vl + v_rd8[dt]));
            const s4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*) (vl + v_rd8[dt] + 16 * 256));
            return s8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        } else {
            const s4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*) (vl + v_rd + dt * 32));
            const s4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*) (vl + v_rd + dt * 32 + 16 * VS));
            return s8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
    };
    auto vread = [&](s8v (&va)[VPRE], const lds_u8* vl) __attribute__((always_inline)) {
#pragma unroll
        for (int dt = 0; dt < VPRE; ++dt) va[dt] = vread1(vl, dt);
    };
    auto scores = [&](f4v (&s)[RT][2], const lds_u8* kl, const s8v (&kpre)[KPRE][KB]) __attribute__((always_inline)) {
        if constexpr (KPRE == 2) {
            // every operand is in registers: the 2 RT chains of dependent products advance side by side
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int kt2 = 0; kt2 < 2; ++kt2)
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt)
                    {
                        s[rt][kt2] = mfma16<BF>(kpre[kt2][kb], qreg[rt][kb], kb == 0 ? ntile[rt] : s[rt][kt2]);
                        if constexpr (QS) s[rt][kt2] = mfma16<BF>(kpre[kt2][kb], qlo[rt][kb], s[rt][kt2]);
                    }
        } else {
#pragma unroll
            for (int kt2 = 0; kt2 < 2; ++kt2) {
                s8v ka[KB];
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
                    ka[kb] = kt2 == 0 ? kpre[0][kb] : *reinterpret_cast<const __attribute__((address_space(3))) s8v*>(kl + k_rd + kt2 * 16 * KS + kb * 64);
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    f4v acc = mfma16<BF>(ka[0], qreg[rt][0], ntile[rt]);
#pragma unroll
                    for (int kb = 1; kb < KB; ++kb) acc = mfma16<BF>(ka[kb], qreg[rt][kb], acc);
                    if constexpr (QS) {
#pragma unroll
                        for (int kb = 0; kb < KB; ++kb) acc = mfma16<BF>(ka[kb], qlo[rt][kb], acc);
                    }
                    s[rt][kt2] = acc;
                }
            }
        }
    };
    // O^T += V^T P^T of one 32-key half (LDS byte offset vl) with the weights in pb
    constexpr short ONE16 = BF ? (short) 0x3F80 : (short) 0x3C00;
    const s8v ones = {ONE16, ONE16, ONE16, ONE16, ONE16, ONE16, ONE16, ONE16};
    auto weigh = [&](const lds_u8* vl, const s8v (&vpre)[VPRE]) __attribute__((always_inline)) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            l4[rt] = mfma16<BF>(ones, pb[rt], l4[rt]);
            if constexpr (BF) l4[rt] = mfma16<BF>(ones, pl[rt], l4[rt]);
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const s8v va = dt < VPRE ? vpre[dt] : vread1(vl, dt);
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                o[rt][dt] = mfma16<BF>(va, pb[rt], o[rt][dt]);
                if constexpr (BF) o[rt][dt] = mfma16<BF>(va, pl[rt], o[rt][dt]);
            }
        }
    };
    // One step of the wave's software pipeline. Step s holds the scores of its own half in sc (computed a step earlier)
    // and runs, as two straight-line blocks in which matrix and vector work are independent and overlap:
    //   A: O^T += V^T P^T of step s - 1   ||   exponent arguments of step s against the reference as it stands, and
    //      this lane's largest
    //   (only if some row's score outgrew its reference by more than 2^8: move the references, rescale; the weights may
    //    otherwise exceed 1, by at most 2^8: harmless in float32 sums and 16-bit operands, and the final division by
    //    the row's sum makes the result the same function of the inputs)
    //   B: S^T of step s + 1              ||   weights of step s = exp2(arguments), rounded to 16 bit
    // Every LDS operand of a block is requested a block ahead (vread at the step's start, kread at the head of A), and
    // sched_group_barrier deals the vector instructions out between the matrix instructions.
    // The mask is applied under a wave-uniform branch: steps no row's causal or window edge crosses pay no comparison.
    auto step = [&](f4v (&sc)[RT][2], f4v (&sn)[RT][2], const lds_u8* kl_next, const lds_u8* vl_prev, int j0, bool masked, bool bar_mid = false) __attribute__((always_inline)) {
        float a[RT][8], amax[RT];
        s8v vpre[VPRE], kpre[KPRE][KB];
        vread(vpre, vl_prev);
        // (the mask goes onto the raw scores: minus infinity stays minus infinity under the positive scale)
        if (masked) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                // keys lo .. hi of this half (relative, clamped into 0 .. 32 / -1 .. 31) are the row's: one unsigned
                // compare a key (no key at all: lo = 64 puts every key below it)
                const int lo_ = std::min(std::max(lo32[rt] - j0, 0), 32);
                const int hi = std::min(std::max(hi32[rt] - j0, -1), 31);
                const int lo = hi < lo_ ? 64 : lo_;
                const unsigned span = hi < lo_ ? 0u : (unsigned) (hi - lo_);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int j = (e >> 2) * 16 + g4 * 4 + (e & 3);
                    sc[rt][e >> 2][e & 3] = (unsigned) (j - lo) <= span ? sc[rt][e >> 2][e & 3] : -INFINITY;
                }
            }
        }
        __builtin_amdgcn_s_setprio(1);
        kread(kpre, kl_next);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int e = 0; e < 8; ++e) a[rt][e] = PRESCALE ? sc[rt][e >> 2][e & 3] : __builtin_fmaf(sc[rt][e >> 2][e & 3], p.sl2, nbr[rt]);
        weigh(vl_prev, vpre);
        bool grow = false;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            amax[rt] = max3f(max3f(max3f(a[rt][0], a[rt][1], a[rt][2]), a[rt][3], a[rt][4]), max3f(a[rt][5], a[rt][6], a[rt][7]), a[rt][7]);
            grow |= amax[rt] > thr[rt];
        }
        if constexpr (D == 128) {
            // the matrix instructions of this block with two vector instructions between each
#pragma unroll
            for (int i = 0; i < (BF ? 2 : 1) * (RT * DT + RT); ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, PRESCALE ? 1 : 2, 0);
            }
        }
        if (bar_mid) tile_barrier();
        if (__any(grow)) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                const float mx = rows_max(amax[rt]);
                const bool fresh = thr[rt] < 0.0f;
                const bool nokey = mx == -INFINITY;
                const float delta = fresh ? (nokey ? 0.0f : mx) : fmaxf(mx, 0.0f);
                const float c = fresh ? 1.0f : fast_exp2(-delta);
                l4[rt] *= c;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) o[rt][dt] *= c;
                nbr[rt] -= delta;
                if constexpr (PRESCALE) ntile[rt] = f4v{nbr[rt], nbr[rt], nbr[rt], nbr[rt]};
#pragma unroll
                for (int e = 0; e < 8; ++e) a[rt][e] -= delta;
                thr[rt] = (fresh && nokey) ? -INFINITY : 8.0f;
            }
        }
        scores(sn, kl_next, kpre);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float pv = fast_exp2(a[rt][e]);                                   // -inf -> 0
                pb[rt][e] = to16<BF>(pv);
                if constexpr (BF) pl[rt][e] = to16<BF>(pv - __builtin_bit_cast(float, (uint32_t) (uint16_t) pb[rt][e] << 16));
            }
        }
        if constexpr (D == 128) {
            // a matrix instruction, an exponential, and a conversion after every other
#pragma unroll
            for (int i = 0; i < RT * 2 * KB; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x400, 1, 0);
                if (i & 1) __builtin_amdgcn_sched_group_barrier(0x002, 1, 0);
            }
        }
        // the step's results are complete here, in program order: nothing of it drifts past the next barrier or branch
        if constexpr (RT == 2) asm volatile("" : "+v"(pb[0]), "+v"(pb[1]));
        else asm volatile("" : "+v"(pb[0]));
        if constexpr (BF && RT == 2) asm volatile("" : "+v"(pl[0]), "+v"(pl[1]));
        else if constexpr (BF) asm volatile("" : "+v"(pl[0]));
        __builtin_amdgcn_s_setprio(0);
    };

    // ---- the pipeline over tiles. K and V tiles have two LDS buffers each (tile k in buffer k & 1) and one register
    // set each; one barrier a tile, between its two steps:
    //   step 2k   : K(k+1) registers -> LDS, fetch K(k+2); A reads V(k-1) half 1, B reads K(k) half 1
    //   barrier
    //   step 2k+1 : V(k+1) registers -> LDS, fetch V(k+2); A reads V(k) half 0,   B reads K(k+1) half 0
    // A wave runs steps sb - 1 .. se of its own (the one before its first computes nothing it keeps except the scores of
    // the first; the one after its last adds the last step's product); all waves take part in the staging of every tile.
    // 8 waves of 128-wide heads: the upper four meet a tile's barrier a block earlier in their own stream - inside the
    // tile's first step, between its product with the values and its scores, whose key operands (and the values') are all
    // in registers by then, so nothing they read later can be overwritten by a wave that is already past the barrier. The
    // two waves of a SIMD then run half a step apart: one asks LDS for its value operands while the other is between
    // reads (config 2: -1 % of the kernel's time)
    const bool upper = D == 128 && PW == 8 && KPRE == 2 && VPRE == DT && w >= PW / 2;
    if (nt > 0) {
        f4v sA[RT][2], sB[RT][2];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int kt2 = 0; kt2 < 2; ++kt2) sA[rt][kt2] = sB[rt][kt2] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
      if constexpr (DMA) {
        // ---- three buffers a stream, tile k in buffer k % 3:
        //   step 2k   : request K(k+2);  A reads V(k-1) half 1, B's operands K(k) half 1
        //   barrier (the upper waves: inside step 2k, see above)
        //   step 2k+1 : request V(k+2);  A reads V(k) half 0,   B's operands K(k+1) half 0
        const std::false_type KEYS;
        const std::true_type VALUES;
        lds_u8* const K0 = (lds_u8*) dk0; lds_u8* const K1 = (lds_u8*) dk1; lds_u8* const K2 = (lds_u8*) dk2;
        lds_u8* const W0 = (lds_u8*) dv0; lds_u8* const W1 = (lds_u8*) dv1; lds_u8* const W2 = (lds_u8*) dv2;
       if constexpr (NBUF == 2) {
        // ---- two buffers a stream, tile k in buffer k % 2; behind tile k's barrier K(k) and V(k - 1) have been read, so
        // K(k + 2) and V(k + 1) are requested into their buffers there and have a tile's time to land:
        //   step 2k   : A reads V(k-1) half 1, B's operands K(k) half 1
        //   barrier (every transfer of this wave has landed: K(k+1), V(k));  request K(k+2), V(k+1)
        //   step 2k+1 : A reads V(k) half 0,   B's operands K(k+1) half 0
        dma(K0, kbase, 0, KEYS);
        dma(W0, vbase, 0, VALUES);
        dma(K1, kbase, 1, KEYS);
        {   // the V buffer step 0 "adds" with zero weights must hold numbers
            const u4v z = {0u, 0u, 0u, 0u};
            for (uint32_t at = (uint32_t) tid * 16; at < (uint32_t) TB; at += PW * 64 * 16)
                *reinterpret_cast<__attribute__((address_space(3))) u4v*>(W1 + at) = z;
        }
        tile_barrier();
        {
            s8v kpre[KPRE][KB];
            kread(kpre, K0);
            scores(sA, K0, kpre);
        }
        // kb / vb: the tile's own buffers; kn: the next tile's keys, vp: the tile before's values (the other buffers)
        auto tile2 = [&](int k, lds_u8* kb, lds_u8* vb, lds_u8* kn, lds_u8* vp) __attribute__((always_inline)) {
            step(sA, sB, kb + 32 * 256, vp + 32 * 256, 64 * k, !(64 * k >= w_full_beg && 64 * k + 32 <= w_full_end));
            tile_barrier();
            dma(kb, kbase, k + 2, KEYS);
            dma(vp, vbase, k + 1, VALUES);
            step(sB, sA, kn, vb, 64 * k + 32, !(64 * k + 32 >= w_full_beg && 64 * k + 64 <= w_full_end));
        };
        for (int k = 0; k < nt; k += 2) {
            tile2(k, K0, W0, K1, W1);
            if (k + 1 >= nt) break;
            tile2(k + 1, K1, W1, K0, W0);
        }
        {
            s8v vpre[VPRE];
            lds_u8* const vl = (((nt - 1) & 1) ? W1 : W0) + 32 * 256;
            vread(vpre, vl);
            weigh(vl, vpre);
        }
       } else {
        dma(K0, kbase, 0, KEYS);
        dma(W0, vbase, 0, VALUES);
        dma(K1, kbase, 1, KEYS);
        dma(W1, vbase, 1, VALUES);
        {   // the V buffer step 0 "adds" with zero weights must hold numbers
            const u4v z = {0u, 0u, 0u, 0u};
            for (uint32_t at = (uint32_t) tid * 16; at < (uint32_t) TB; at += PW * 64 * 16)
                *reinterpret_cast<__attribute__((address_space(3))) u4v*>(W2 + at) = z;
        }
        tile_barrier();
        {
            s8v kpre[KPRE][KB];
            kread(kpre, K0);
            scores(sA, K0, kpre);
        }
        // one tile: its two steps; kb / vb: the tile's own buffers, kn: the next tile's keys, vp: the tile before's values,
        // k2 / v2: where the tile after the next goes
        auto tile = [&](int k, lds_u8* kb, lds_u8* vb, lds_u8* kn, lds_u8* vp, lds_u8* k2, lds_u8* v2) __attribute__((always_inline)) {
            dma(k2, kbase, k + 2, KEYS);
            step(sA, sB, kb + 32 * 256, vp + 32 * 256, 64 * k, !(64 * k >= w_full_beg && 64 * k + 32 <= w_full_end), upper);
            if (!upper) tile_barrier();
            dma(v2, vbase, k + 2, VALUES);
            step(sB, sA, kn, vb, 64 * k + 32, !(64 * k + 32 >= w_full_beg && 64 * k + 64 <= w_full_end));
        };
        for (int k = 0; k < nt; k += 3) {
            tile(k, K0, W0, K1, W2, K2, W2);
            if (k + 1 >= nt) break;
            tile(k + 1, K1, W1, K2, W0, K0, W0);
            if (k + 2 >= nt) break;
            tile(k + 2, K2, W2, K0, W1, K1, W1);
        }
        // the last step's product
        {
            s8v vpre[VPRE];
            lds_u8* const vl = ((nt - 1) % 3 == 0 ? W0 : (nt - 1) % 3 == 1 ? W1 : W2) + 32 * 256;
            vread(vpre, vl);
            weigh(vl, vpre);
        }
       }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");           // (transfers past the last tile land in buffers the output goes through)
      } else {
        Stage stk, stv;
        fetch(stk, kbase, 0);
        fetch(stv, vbase, 0);
        {   // the V buffer step 0 "adds" with zero weights must hold numbers
            const u4v z = {0u, 0u, 0u, 0u};
            for (uint32_t at = (uint32_t) tid * 16; at < (uint32_t) VBUF; at += PW * 64 * 16)
                *reinterpret_cast<__attribute__((address_space(3))) u4v*>(L + V0 + VBUF + at) = z;
        }
        stash_k(stk, 0);
        stash_v(stv, 0);
        fetch(stk, kbase, 1);
        fetch(stv, vbase, 1);
        __syncthreads();
        {
            s8v kpre[KPRE][KB];
            kread(kpre, L);
            scores(sA, L, kpre);
        }
        for (int k = 0; k < nt; k += 2) {
            // tile k: buffers 0
            stash_k(stk, 1);
            fetch(stk, kbase, k + 2);
            step(sA, sB, L + 32 * KS, L + V0 + VBUF + 32 * VS, 64 * k, !(64 * k >= w_full_beg && 64 * k + 32 <= w_full_end), upper);
            if (!upper) __syncthreads();
            stash_v(stv, 1);
            fetch(stv, vbase, k + 2);
            step(sB, sA, L + KBUF, L + V0, 64 * k + 32, !(64 * k + 32 >= w_full_beg && 64 * k + 64 <= w_full_end));
            if (k + 1 >= nt) break;
            // tile k + 1: buffers 1
            stash_k(stk, 0);
            fetch(stk, kbase, k + 3);
            step(sA, sB, L + KBUF + 32 * KS, L + V0 + 32 * VS, 64 * k + 64, !(64 * k + 64 >= w_full_beg && 64 * k + 96 <= w_full_end), upper);
            if (!upper) __syncthreads();
            stash_v(stv, 0);
            fetch(stv, vbase, k + 3);
            step(sB, sA, L, L + V0 + VBUF, 64 * k + 96, !(64 * k + 96 >= w_full_beg && 64 * k + 128 <= w_full_end));
        }
        // the last step's product
        {
            s8v vpre[VPRE];
            lds_u8* const vl = L + V0 + (uint32_t) ((nt - 1) & 1) * VBUF + 32 * VS;
            vread(vpre, vl);
            weigh(vl, vpre);
        }
      }
    }

    // ---- out = O / l. A lane holds dims 16 dt + 4 g4 .. + 3 of its rows: the wave's 32 x D block goes through LDS (the
    // tile buffers, free now) so that it leaves as whole rows, 16 bytes a lane and 4 (float32: 2) rows an instruction
    __syncthreads();                                              // every wave is done with the tiles
    // (DMA: the tile buffers are arrays of their own; two waves' staging regions go through each of the first four)
    lds_u8* const OB = DMA && NBUF == 2 ? (w == 0 ? (lds_u8*) dk0 : w == 1 ? (lds_u8*) dk1 : w == 2 ? (lds_u8*) dv0 : (lds_u8*) dv1)
                       : DMA ? ((w & 3) == 0 ? (lds_u8*) dk0 : (w & 3) == 1 ? (lds_u8*) dk1 : (w & 3) == 2 ? (lds_u8*) dk2 : (lds_u8*) dv0) + (w >> 2) * 16 * (D * 4 + 16)
                           : L + w * 16 * (D * 4 + 16);
    if (p.ns > 1) {
        // ---- a key split's partial: the rows' unnormalized sums as float32, then (m, l) - D + 2 floats a (row, head, split),
        // rows 8 bytes aligned: 8-byte pieces, 8 rows an instruction
        const uint32_t rowp = D * 4 + 16;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const float lsum = l4[rt][0];
            const uint32_t at = (uint32_t) n * rowp + (uint32_t) (g4 * 16);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<__attribute__((address_space(3))) f4v*>(OB + at + dt * 64) = o[rt][dt];
            const int row = wbase + rt * 16 + n;
            if (g4 == 0 && row < p.T) {
                float* pr = p.part + (((int64_t) row * p.Hq + hq) * p.ns + split) * (D + 2);
                *reinterpret_cast<float2*>(pr + D) = float2{thr[rt] < 0.0f ? -INFINITY : -nbr[rt], lsum};
            }
            for (int c = lane; c < 16 * (D / 2); c += 64) {
                const int rl_ = c / (D / 2), piece = c % (D / 2), prow = wbase + rt * 16 + rl_;
                if (prow < p.T) {
                    typedef uint32_t u2v __attribute__((ext_vector_type(2)));
                    const u2v x = *reinterpret_cast<const __attribute__((address_space(3))) u2v*>(OB + (uint32_t) rl_ * rowp + (uint32_t) piece * 8);
                    *reinterpret_cast<u2v*>(p.part + (((int64_t) prow * p.Hq + hq) * p.ns + split) * (D + 2) + piece * 2) = x;
                }
            }
        }
        return;
    }
    {
        const int esz = p.qt == 0 ? 4 : 2;
        const uint32_t rowb = (uint32_t) (D * esz), rowp = rowb + 16;    // bytes a row, padded in LDS
        const int ppr = (int) rowb / 16;                          // 16-byte pieces a row
        uint8_t* const orow = reinterpret_cast<uint8_t*>(p.out) + (int64_t) hq * rowb;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const float lsum = l4[rt][0];
            const float inv = lsum > 0.0f ? 1.0f / lsum : 0.0f;
            const uint32_t at = (uint32_t) n * rowp + (uint32_t) (g4 * 4 * esz);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const f4v v = o[rt][dt] * inv;
                if (p.qt == 0) {
                    *reinterpret_cast<__attribute__((address_space(3))) f4v*>(OB + at + dt * 64) = v;
                } else {
                    typedef uint16_t us4v __attribute__((ext_vector_type(4)));
                    us4v h;
                    if (p.qt == 1) h = us4v{f32_to_f16(v[0]), f32_to_f16(v[1]), f32_to_f16(v[2]), f32_to_f16(v[3])};
                    else h = us4v{f32_to_bf16(v[0]), f32_to_bf16(v[1]), f32_to_bf16(v[2]), f32_to_bf16(v[3])};
                    *reinterpret_cast<__attribute__((address_space(3))) us4v*>(OB + at + dt * 32) = h;
                }
            }
            // the wave reads back its own block only: no barrier, the LDS queue keeps a wave's accesses in order
            for (int c = lane; c < 16 * ppr; c += 64) {
                const int rl_ = c / ppr, piece = c % ppr, row = wbase + rt * 16 + rl_;
                if (row < p.T) {
                    const u4v x = *reinterpret_cast<const __attribute__((address_space(3))) u4v*>(OB + (uint32_t) rl_ * rowp + (uint32_t) piece * 16);
                    *reinterpret_cast<u4v*>(orow + (int64_t) row * p.Hq * rowb + piece * 16) = x;
                }
            }
        }
    }
}

// A bfloat16 cache's rows on their way to half rows in position order: positions [kf, kf + n) of every key head, out of a
// cache of any geometry (head-major, position-major, a ring) into [which][head][n][D]. Every bfloat16 value whose
// magnitude lies in half's normal range is a half exactly; larger ones saturate at 65504 (the reference's caches are
// half: kernels/llm/qwen35/q35.cpp:573-588 rounds float32 rows into them), smaller ones round to half's subnormals.
struct WidenParams {
    const uint8_t* src[2];
    uint8_t* dst[2];
    int64_t head_stride, row_stride, cap, kf, n;
    int wrap;
};
template <int CPR>   // 16-byte chunks a row: D / 8
__global__ __launch_bounds__(256) void kv_bf16_to_half_kernel(const WidenParams p) {
    const int64_t j = (int64_t) blockIdx.x * (256 / CPR) + threadIdx.x / CPR;
    const int c = threadIdx.x % CPR, h = blockIdx.y, z = blockIdx.z;
    if (j >= p.n) return;
    const int64_t pos = p.kf + j, slot = p.wrap ? pos % p.cap : pos;
    const u4v x = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(p.src[z] + h * p.head_stride + slot * p.row_stride + c * 16));
    u4v y;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float lo = fminf(fmaxf(__builtin_bit_cast(float, x[i] << 16), -65504.0f), 65504.0f);
        const float hi = fminf(fmaxf(__builtin_bit_cast(float, x[i] & 0xFFFF0000u), -65504.0f), 65504.0f);
        y[i] = (uint32_t) __builtin_bit_cast(uint16_t, (_Float16) lo) | ((uint32_t) __builtin_bit_cast(uint16_t, (_Float16) hi) << 16);
    }
    *reinterpret_cast<u4v*>(p.dst[z] + (((int64_t) h * p.n + j) * CPR + c) * 16) = y;
}

// The same for q8_0 (KT = 1) and q4_0 (KT = 2) rows: a thread takes 8 values of a 32-value block - 8 bytes, or one nibble
// of each of 8 bytes - and writes the 8 halfs the kernels' own staging makes of them (half(q x d), one rounding: dq8x8 /
// dq4x8), so the pass over the widened rows sees the operands the pass over the raw rows would have built.
template <int KT, int CPR>   // 8-value chunks a row: D / 8
__global__ __launch_bounds__(256) void kv_quant_to_half_kernel(const WidenParams p) {
    constexpr int D = CPR * 8;
    const int64_t j = (int64_t) blockIdx.x * (256 / CPR) + threadIdx.x / CPR;
    const int c = threadIdx.x % CPR, h = blockIdx.y, z = blockIdx.z;
    if (j >= p.n) return;
    const int64_t pos = p.kf + j, slot = p.wrap ? pos % p.cap : pos;
    const uint8_t* const row = p.src[z] + h * p.head_stride + slot * p.row_stride;
    const int b = c / 4, cc = c % 4;
    dq_s8v y;
    if constexpr (KT == 1) {
        const uint2 x = *reinterpret_cast<const uint2*>(row + c * 8);
        y = dq8x8(x.x, x.y, __builtin_bit_cast(_Float16, *reinterpret_cast<const uint16_t*>(row + D + 2 * b)));
    } else {
        const uint2 x = *reinterpret_cast<const uint2*>(row + b * 16 + (cc & 1) * 8);
        y = dq4x8(x.x, x.y, cc >= 2 ? 4 : 0, __builtin_bit_cast(_Float16, *reinterpret_cast<const uint16_t*>(row + D / 2 + 2 * b)));
    }
    *reinterpret_cast<dq_s8v*>(p.dst[z] + (((int64_t) h * p.n + j) * CPR + c) * 16) = y;
}

// Query heads a work-group holds (PrefillParams::pack): a pass of so few rows that they fill only some of a work-group's
// waves gives the other waves further heads of the same key head - 32 rows and fewer: 4 heads to 4 waves - and every
// staged tile then serves them all (17 rows x 32 / 8 heads behind 32768 keys: each head's work-group re-staged the keys
// for one live wave). A divisor of the group: 5 heads take 5 of 8 waves.
int64_t pack_of(int64_t T, int64_t G, int64_t D, int64_t PW) {
    const int64_t need = (T + (D == 128 ? 32 : 16) - 1) / (D == 128 ? 32 : 16);       // waves the rows of one head fill
    int64_t pack = 1;
    for (int64_t c = 2; c * need <= PW; ++c)
        if (G % c == 0) pack = c;
    return pack;
}

// Whether a pass over rows that are not half keeps their form in the kernel instead of widening them to half rows first
// (knob 5 = 0: the measured rule). What widening costs is read and written once a key; a pass of few rows reads a key
// only once a row block and query head of its group, and the kernel's own staging of it is then the shorter way. T rows x
// G heads a key head behind `keys` keys, float32 query rows, widened / own form in us:
//   bfloat16 (bfloat16 query rows up to 128 rows x D / 32 heads; rows of another type, which enter the first product in
//     two parts - twice its matrix instructions - up to 2 D rows a key head; behind fewer than 4096 keys the widening
//     costs next to nothing and its pass is the shorter): 64 x 4 of 128 behind 32768 keys 107 / 84, 17 x 4 behind 131072
//     333 / 164, 128 x 4 behind 32768 120 / 122; 17 bfloat16 rows x 1 behind 2048 35 / 38
//   q8_0 rows of 128 behind 32768 keys and more, up to 8 reads a key: 17 x 4 behind 131072 294 / 158, 128 x 4 behind
//     32768 111 / 86, 64 x 4 behind 8192 42 / 54; 17 x 16 behind 131072 217 / 215. Rows of 256 behind 65536 keys and
//     more, up to 256 rows a key head: 17 x 4 behind 131072 130 / 86, 32 x 8 154 / 139, 64 x 8 220 / 240; 17 x 8 behind
//     32768 54 / 62
//   q4_0 rows of 128 up to 1024 rows a key head: 64 x 4 behind 32768 92 / 67, 17 x 16 behind 131072 214 / 157, 128 x 16
//     behind 32768 143 / 148. Rows of 256 behind 32768 keys and more, up to 8 reads a key: 64 x 8 behind 131072 217 /
//     176, 17 x 8 there 147 / 95, 17 x 8 behind 8192 36 / 43
bool own_form_pays(int kt, int qt, int64_t D, int64_t T, int64_t G, int64_t keys) {
    const int64_t key_reads = ((T + 127) / 128) * G;
    switch (kt) {
        case 3: return keys >= 4096 && key_reads <= D / 32 && (qt == 2 || T * G <= 2 * D);
        case 1: return D == 128 ? keys >= 32768 && key_reads <= 8 : keys >= 65536 && T * G <= 256;
        case 2: return D == 128 ? T * G <= 1024 : keys >= 32768 && key_reads <= 8;
        default: return false;
    }
}

template <int D, int PW>
int launch_prefill(ns_gpu* g, int kt, const PrefillParams& p, dim3 grid, bool stream) {
    constexpr int TH = PW * 64;
    if constexpr (D == 128) {
        // (the streaming forms: half rows with either work-group size, bfloat16 rows - short passes keep them - with 4 waves)
        if (stream && kt == 0) {
            attn_prefill_kernel<D, false, 0, PW, false, true><<<grid, TH, 0, g->q>>>(p);
            return 0;
        }
        if constexpr (PW == 4) {
            if (stream && kt == 3) {
                if (p.qt != 2) attn_prefill_kernel<D, true, 0, PW, true, true><<<grid, TH, 0, g->q>>>(p);
                else attn_prefill_kernel<D, true, 0, PW, false, true><<<grid, TH, 0, g->q>>>(p);
                return 0;
            }
        }
    }
    if (kt == 0) {
        attn_prefill_kernel<D, false, 0, PW><<<grid, TH, 0, g->q>>>(p);
    } else if (kt == 3) {
        if (p.qt != 2) attn_prefill_kernel<D, true, 0, PW, true><<<grid, TH, 0, g->q>>>(p);
        else attn_prefill_kernel<D, true, 0, PW><<<grid, TH, 0, g->q>>>(p);
    } else if (kt == 1) {
        attn_prefill_kernel<D, false, 1, PW><<<grid, TH, 0, g->q>>>(p);
    } else if constexpr (D == 256 || PW == 4) {
        attn_prefill_kernel<D, false, 2, PW><<<grid, TH, 0, g->q>>>(p);
    } else {
        // (a q4_0 tile of 128-value rows is 256 chunks: fewer than 8 waves have threads - the caller takes 4 waves)
        return ns_fail("ns_attn_prompt: internal: q4_0 rows of 128 values take 4 waves");
    }
    return 0;
}


}  // namespace

int ns_attn_prompt_any(ns_gpu* g, const char* who, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T,
                       int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, int causal, int64_t kfirst, float scale,
                       void* out) {
    NS_TRY
    const std::string w(who);
    if (T <= 0) return 0;
    if (D != 128 && D != 256) return ns_fail(w + ": heads of 128 or 256");
    if (Hkv <= 0 || Hq <= 0 || Hq % Hkv) return ns_fail(w + ": query heads a multiple of the key heads");
    if (kt < 0 || kt > 3) return ns_fail(w + ": a cache form 0 (half), 1 (q8_0), 2 (q4_0) or 3 (bfloat16)");
    if (qt < 0 || qt > 2) return ns_fail(w + ": rows of type 0 (float32), 1 (half) or 2 (bfloat16)");
    if (p0 < 0 || cap <= 0 || win < 0) return ns_fail(w + ": a position, a capacity and a window of 0 or more");
    if (kfirst > p0) return ns_fail(w + ": a block's first key lies at or before its first row");
    const int64_t need = pm ? p0 + T : (win > 0 ? std::min(p0 + T, win + T - 1) : p0 + T);
    if (need > cap) return ns_fail(w + (win > 0 ? ": the cache's ring is shorter than the window and the pass" : ": past the cache's capacity"));
    if (!q || !kc || !vc || !out) return ns_fail(w + ": a null buffer");
    if ((uintptr_t) q % 16 || qs % (qt == 0 ? 4 : 8) || (uintptr_t) out % 16) return ns_fail(w + ": query and output rows 16-byte aligned");
    const int64_t rb = kv_row_bytes(kt, D);
    // rows are fetched in 16-byte chunks: every 16-bit row keeps that alignment, q8_0 / q4_0 rows do at D = 256 (272 / 144
    // bytes; the reference's quantized prompt form is D = 256 only); at D = 128 (136 / 72 bytes) the chunks are 8-byte aligned
    if (((uintptr_t) kc | (uintptr_t) vc) % (rb % 16 ? 8 : 16)) return ns_fail(w + (rb % 16 ? ": caches 8-byte aligned" : ": caches 16-byte aligned"));
    // (512 work-groups of 256 rows: two for each of the chip's 256 CUs; NS_PREFILL_WAVES = 4 or 8 overrides: tuning, tests)
    int64_t sns = 1, skbs = 0, sk0 = 0;
    // heads a work-group of a short pass holds (pack_of): with 4 waves, or - where only 8 waves let a group share at all,
    // 5 or 7 heads - with 8
    const int64_t pk4 = pack_of(T, Hq / Hkv, D, 4), pk8 = pack_of(T, Hq / Hkv, D, 8);
    const bool wide_pack = pk8 > 2 * pk4 && (pk4 == 1 || p0 + T >= 8192);     // (a group that shares with 4 waves too: only behind a long context)
    // (heads of 256, up to 64 rows behind a long context: 8 waves - twice the heads a work-group, and one work-group a CU
    // is all its LDS admits - 17 rows x 16 / 2 heads behind 131072 keys 130 -> 92 us)
    const bool long256 = D == 256 && T <= 64 && p0 + T >= 16384;
    const int64_t pkp = wide_pack || long256 ? pk8 : pk4;
    // Key splits. A pass of few rows over a long context - a chunk of a prompt behind 32K tokens, a long draft block - has
    // too few (row block, head) pairs to fill the chip, each walking every key: its keys are cut into ns splits of whole
    // tiles, a work-group a (row block, head, split), the partials merged by the decode path's merge kernel. ns is
    // decided from the pass alone (128-row blocks x heads against ~512 work-groups; splits no shorter than the context's length warrants), not
    // from the work-group size, so both sizes sum a row in the same order. The partials live in the library's own
    // scratch (the prompt entry points have no scratch argument): what fits bounds ns.
    {
        const int64_t kf = kfirst >= 0 ? kfirst : win > 0 ? std::max<int64_t>(0, p0 + 1 - win) : 0, keys = p0 + T - kf;
        const int64_t pairs = ((T + 127) / 128) * Hq / pkp;
        // (how far a context is worth cutting grows with its root where the (row block, head) pairs are few - under 32:
        // splits of about 256 keys at 2048, 512 at 8192, 1024 at 32768, 2048 at 131072; shorter ones cost more in partials
        // and their merge than they save, longer ones leave a work-group a long chain of tiles; under 512 keys none. Up to
        // 64 pairs: twice that; more: 1024 keys and more. 17 rows x 32 / 8 heads behind 1024 keys 25.3 -> 17.5 us, behind 2048
        // 28.1 -> 20.2, behind 8192 32.8 -> 29.7; 128 rows behind 2048 keys 30.8 -> 26.1.
        // A pass about as long as its context is mostly diagonal - its row blocks see different key counts, and equal cuts
        // of the keys leave them unequal work - and is cut as a long pass is, by 1024 keys; so is a pass whose work-groups
        // hold one head's few rows, three waves of four idle: 17 rows x 40 / 8 heads behind 8192 keys 42 us in 8 splits, 49 in 13)
        const bool filled = pkp > 1 || T > (D == 128 ? 64 : 32);      // (rows for three of 4 waves of 32 rows, or of 16)
        const int64_t root = keys < 512 ? 1 : (int64_t) (0.177 * std::sqrt((double) keys));
        // (few pairs: at least the splits that give every CU a work-group, down to a tile or 2 T keys a split - the partials
        // grow with the rows - 17 rows x 8 / 1 heads behind 32768 keys in 32 splits 30.0 us, in 128 20.3; 32 / 8 heads behind
        // 8192 keys in 16 24.7, in 32 21.3; 17 rows x 4 / 4 heads, a head's few rows a work-group, behind 8192 keys in 8
        // 32.4, in 64 15.4. Heads of 256 - one work-group a CU - take exactly those: 40 rows x 16 / 2 heads behind 131072
        // keys in 32 splits 163 us, in 64 175)
        const int64_t fill = keys < 512 ? 1 : std::min<int64_t>((256 + pairs - 1) / pairs, keys / std::max<int64_t>(KT_TILE, 2 * T));
        const int64_t by_keys = p0 < 2 * T || pairs > 64 ? keys / 1024
                                : pairs < 32         ? (D == 256 ? std::max<int64_t>(fill, 1) : std::max(root, fill))
                                : !filled            ? keys / 1024
                                                     : std::max(keys / 1024, root / 2);
        const int64_t aim = 512;
        int64_t ns = std::min<int64_t>({(aim + pairs - 1) / pairs, by_keys, 128,
                                        (int64_t) (ns_own_floats(g) / (size_t) (T * Hq * (D + 2)))});
        // (a pass the context dominates - equal work-groups - whose count would fill the chip's 512 places unevenly, say 640:
        // cut further, to about two and a half rounds. 1024 rows x 40 heads behind 32768 keys: 740 -> 652 us; 2048 rows: 1467 -> 1280)
        // (a pass of few pairs whose splits overfill a round of the chip's places - heads of 256: one work-group a CU; 24
        // heads x 16 splits = a round and a half - is cut into fewer, to whole rounds: 33 rows x 24 / 4 heads of 256 behind
        // 8192 keys 59 -> 45 us)
        {
            const int64_t slots = D == 128 ? 512 : 256, wg = pairs * std::max<int64_t>(ns, 1);
            if (ns > 1 && wg > slots && wg <= 2 * slots && 100 * wg < 85 * ((wg + slots - 1) / slots * slots)) ns = std::max<int64_t>(1, slots / pairs);
        }
        if (p0 >= T && keys / 1024 >= 2) {
            const int64_t slots = D == 128 ? 512 : 256;
            const int64_t cap_ns = std::min<int64_t>({keys / 1024, 64, (int64_t) (ns_own_floats(g) / (size_t) (T * Hq * (D + 2)))});
            auto fill_of = [&](int64_t n) { const int64_t w = pairs * n; return (double) w / (double) ((w + slots - 1) / slots * slots); };
            if (fill_of(std::max<int64_t>(ns, 1)) < 0.85) ns = std::max(ns, std::min<int64_t>((5 * slots / 2 + pairs - 1) / pairs, cap_ns));
            // (and from there the count - up to three more - whose rounds are fullest, a split more charged what its
            // partials cost against the pass, 620 / keys: 5000 rows x 32 heads behind 32768 keys are 1280 work-groups, two
            // rounds and a half; in two splits five whole ones: 2657 -> 2505 us, x 40 heads 3613 -> 3178)
            const int64_t from = std::max<int64_t>(ns, 1);
            if (p0 >= 2 * T && fill_of(from) < 0.92) {      // (behind less than two passes' keys the diagonal makes the work-groups unequal)
                double best = 0.0;
                for (int64_t n = from; n <= std::min(from + 3, std::max(cap_ns, from)); ++n) {
                    const double fill = fill_of(n) - 620.0 / (double) keys * (double) (n - from);
                    if (n == from || fill > best + 0.02) best = fill, ns = n;
                }
            }
        }
        // (a forced count - tests - stays within what the scratch and the merge kernel hold)
        if (const int64_t forced = ns_tune_get(NS_TUNE_PREFILL_SPLITS)) ns = std::min<int64_t>({forced, 2048, (int64_t) (ns_own_floats(g) / (size_t) (T * Hq * (D + 2)))});
        if (ns >= 2) {
            sk0 = kf / KT_TILE * KT_TILE;
            skbs = ((p0 + T - sk0 + ns - 1) / ns + KT_TILE - 1) / KT_TILE * KT_TILE;
            sns = (p0 + T - sk0 + skbs - 1) / skbs;
        }
    }
    // head size 256, 16-bit rows: a wave owns one 16-row tile, so 8 waves (two a SIMD, 128-row blocks) run the job 1.5 x
    // as fast as 4 (one a SIMD) whenever there are blocks enough for half the CUs
    // (heads of 128: 256-row blocks pay only where whole ones fill the chip twice over; a pass cut into key splits has few rows -
    // 64 rows x 64 heads behind 32768 keys: 476 us in 256-row blocks that are three quarters empty, 267 us in 128-row ones;
    // 256 rows: 518 against 308)
    // A cache that is not half is widened first when its rows fit the library's scratch behind the partials (below)
    const int64_t wkf = kfirst >= 0 ? kfirst : win > 0 ? std::max<int64_t>(0, p0 + 1 - win) : 0, wn = p0 + T - wkf;
    const size_t part_bytes = sns > 1 ? ((size_t) (T * Hq * sns * (D + 2)) * 4 + 255) / 256 * 256 : 0;
    const size_t wone = (size_t) (Hkv * wn * D * 2);
    const bool own_form = ns_tune_get(NS_TUNE_PREFILL_BF16) == 1 || (ns_tune_get(NS_TUNE_PREFILL_BF16) == 0 && own_form_pays(kt, qt, D, T, Hq / Hkv, wn));
    const bool widen = kt != 0 && !own_form && part_bytes + 2 * wone <= ns_own_floats(g) * 4 && wn * D * 2 < (int64_t) 1 << 32;
    int PWs = D == 128 ? (sns == 1 && ((T + 255) / 256) * Hq >= 512 ? 8 : 4) : (T > 64 && ((T + 127) / 128) * Hq * sns >= 128 ? 8 : 4);
    // (a pass cut into key splits takes 8 waves after all where its rows - some heads of them to a work-group - fill
    // every 256-row block to 70 % and the blocks the chip, one a CU: a staged tile then serves twice the rows. 128 rows x 64 / 4
    // heads behind 32768 keys 142 -> 131 us, 256 rows 260 -> 240; x 32 / 8 heads 192 rows 141 -> 130)
    // (heads of 256: 33 - 64 rows behind a long context - 128 rows of two heads to an 8-wave work-group, one staging of the
    // keys for both - 16 / 2 heads behind 32768 keys 92 -> 70 us, 32 / 8 heads 131 -> 94; behind 8192 keys the 4-wave form)
    if (long256 && sns > 1) PWs = 8;
    if (D == 128 && sns > 1 && T >= 96) {
        const int64_t rb8 = (8 / pk8) * 32, blocks8 = (T + rb8 - 1) / rb8;
        const int64_t last8 = T - (blocks8 - 1) * rb8, wg8 = blocks8 * (Hq / pk8) * sns;
        // (the last block filled like the others - 384 rows = a block and a half: 233 -> 286 us - and whole rounds of the
        // 256 CUs - 520 work-groups, 40 heads x 13 splits, are three rounds: 74 -> 80 us)
        if (10 * last8 >= 7 * rb8 && wg8 >= 256 && 100 * wg8 >= 85 * ((wg8 + 255) / 256 * 256)) PWs = 8;
    }
    if (wide_pack) PWs = 8;
    if (const int64_t forced = ns_tune_get(NS_TUNE_PREFILL_WAVES); forced == 4 || forced == 8) PWs = (int) forced;
    if (kt == 2 && D == 128 && !widen) PWs = 4;                              // (a q4_0 tile of 128-value rows has chunks for 256 threads)
    const int64_t ROWS = rows_of((int) D, PWs);
    if (T > (int64_t) 1 << 30 || ((T + ROWS - 1) / ROWS + 1) * Hq > (int64_t) 1 << 30) return ns_fail(w + ": too many rows or heads");
    if ((pm ? cap * Hkv : cap) * rb >= (int64_t) 1 << 32) return ns_fail(w + ": a key head's cache spans 4 GiB or more");
    NS_HIP(hipSetDevice(g->dev));
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
    p.causal = causal;
    p.kfirst = kfirst;
    p.sl2 = (scale > 0.0f ? scale : 1.0f / sqrtf((float) D)) * 1.4426950408889634f;
    p.out = out;
    p.ns = (int) sns;
    p.kbs = skbs;
    p.k0 = sk0;
    p.part = g->own_scratch;
    // A cache that is not half. As bfloat16 operands the softmax weights carry 8 significant bits each - the kernel then
    // enters them as two numbers, twice the second product's matrix instructions - query rows of another type are rounded
    // to 8 bits, and the query cannot take the scale (a second rounding at 8 bits shows); q8_0 / q4_0 rows are staged as
    // halfs by every work-group that reads them, once a row block and query head. So the pass's key and value rows are
    // first widened to half (bfloat16 exactly, quantized rows to the halfs the kernel's own staging builds) into the
    // library's scratch, behind the key splits' partials, and the pass runs as one over a half cache: half weights and a
    // scaled half query, as in the reference's kernels (8192 rows behind 32768 keys, rows of 256: q8_0 7062 -> 4827 us,
    // q4_0 5288 -> 4742, bfloat16 5963 -> 4666). A pass whose rows do not fit the scratch keeps the rows' own form.
    int kt_run = kt;
    if (widen) {
        {
            const int64_t kf = wkf, n = wn;
            const size_t one = wone;
            uint8_t* const buf = (uint8_t*) g->own_scratch + part_bytes;
            WidenParams wp{};
            wp.src[0] = (const uint8_t*) kc;
            wp.dst[0] = buf;
            wp.src[1] = (const uint8_t*) vc;
            wp.dst[1] = buf + one;
            wp.head_stride = p.head_stride;
            wp.row_stride = p.row_stride;
            wp.cap = cap;
            wp.kf = kf;
            wp.n = n;
            wp.wrap = p.wrap;
            const dim3 wgrid((unsigned) ((n * (D / 8) + 255) / 256), (unsigned) Hkv, 2u);
            if (kt == 3) {
                if (D == 128) kv_bf16_to_half_kernel<16><<<wgrid, 256, 0, g->q>>>(wp);
                else kv_bf16_to_half_kernel<32><<<wgrid, 256, 0, g->q>>>(wp);
            } else if (kt == 1) {
                if (D == 128) kv_quant_to_half_kernel<1, 16><<<wgrid, 256, 0, g->q>>>(wp);
                else kv_quant_to_half_kernel<1, 32><<<wgrid, 256, 0, g->q>>>(wp);
            } else {
                if (D == 128) kv_quant_to_half_kernel<2, 16><<<wgrid, 256, 0, g->q>>>(wp);
                else kv_quant_to_half_kernel<2, 32><<<wgrid, 256, 0, g->q>>>(wp);
            }
            NS_LAUNCHED("kv_to_half");
            // (position j of head h at buf + (h n + j - kf) 2 D: the kernel is given the address position 0 would have)
            p.kc = buf - kf * D * 2;
            p.vc = buf + one - kf * D * 2;
            p.head_stride = n * D * 2;
            p.row_stride = D * 2;
            p.wrap = 0;
            kt_run = 0;
        }
    }
    p.pack = (int) pack_of(T, Hq / Hkv, D, PWs);
    p.gw = (int) (Hq / Hkv) / p.pack;
    const int64_t RB = (PWs / p.pack) * (ROWS / PWs);
    const int64_t units = ((T + RB - 1) / RB) * Hkv * p.ns;            // (split, row block, key head); padded to the 8 XCDs
    if ((units + 7) / 8 * 8 * p.gw >= (int64_t) 1 << 31) return ns_fail(w + ": too many work-groups");
    dim3 grid((unsigned) ((units + 7) / 8 * 8 * p.gw));
    if (ns_profile_mark(g, 0)) return -1;
    // (a pass whose keys are each read by one work-group - all the group's heads in it, one row block - behind a long
    // context streams them: 17 rows x 32 / 8 heads behind 131072 keys 110 -> 97 us; where several work-groups read a key
    // the streaming policy loses what they share in L2: x 64 / 4 heads 142 -> 156)
    const bool stream = p.gw == 1 && T <= RB && p0 + T >= 32768;
    if ((D == 256 ? (PWs == 8 ? launch_prefill<256, 8>(g, kt_run, p, grid, false) : launch_prefill<256, 4>(g, kt_run, p, grid, false))
                  : PWs == 8 ? launch_prefill<128, 8>(g, kt_run, p, grid, stream) : launch_prefill<128, 4>(g, kt_run, p, grid, stream)) != 0)
        return -1;
    NS_LAUNCHED("attn_prefill");
    if (ns_profile_mark(g, 1)) return -1;
    if (p.ns > 1) {
        if (ns_attn_merge_partials(g, D, p.part, p.ns, qt, T * Hq, out)) return -1;
        return ns_profile_mark(g, 2);
    }
    return 0;
    NS_CATCH
}

extern "C" {

int ns_attn_prompt_t(ns_gpu* g, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq,
                     int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, float scale, void* out) {
    return ns_attn_prompt_any(g, "ns_attn_prompt_t", qt, kt, pm, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, win, 1, -1, scale, out);
}

}  // extern "C"
