// attn_decode.hip: split-K GQA decode / verify attention over the KV cache (half, bfloat16, q8_0, q4_0 rows) for gfx950.
//
// Bound: HBM. A decode pass reads every visible key and value once (2 x row bytes a key and key head) and computes
// 4 D flops a (row, key): at most 32 flop/byte for a 4-row verify pass - far under the MFMA ridge, so the kernel is
// built to keep HBM reads in flight and everything else out of their way.
//
// Work split: grid (key split, key head, row chunk). A work-group of 4 waves owns the keys [s kbs, (s + 1) kbs) of one
// key head - kbs a multiple of 128 chosen so the grid has ~NS_DEC_WGS work-groups whatever the context - and ALL the
// pass's T x G query rows of that key head ride on every key tile, so a key is read from HBM once. Wave w takes the
// 32-key tiles with (tile index % 4 == w): tiles and splits sit at absolute key positions, which (with MFMA columns
// being independent) makes a row's arithmetic the same whatever rows share its pass - the verify invariant.
//
// A wave's tile step (32 keys), all in the transposed orientation so no row statistic ever crosses lanes through LDS:
//   K:  half / bfloat16 rows: global -> LDS directly, read back as the MFMA A operand (ds_read_b128: lane = key, 16
//       bytes of its row per k-block); q8_0 rows and q4_0 rows of 256: the raw rows global -> LDS, lifted into registers
//       and widened to half there; q4_0 rows of 128: global -> registers
//   S^T[key][row] = K Q^T           v_mfma_f32_16x16x32 (rows padded to 16-row tiles; Q^T lives in registers)
//   online softmax, base 2, float32: a lane holds 8 keys of one row; row max / sum = 8 in-lane + 2 xor-shuffles
//   P^T -> 16 bit: it already IS the B operand of the next product (k-slot i of lane group g <-> key 4 g + i | 16 + 4 g + i)
//   V:  half / bfloat16 rows: global -> LDS directly (global_load_lds_dwordx4, 1 KiB contiguous per instruction), the
//       16-byte chunks of a row XOR-swizzled by the key so the transposing reads meet no bank conflicts; q8_0 / q4_0
//       rows: lifted as the keys are, widened to half in registers -> LDS [key][D] (rows padded by 32 bytes);
//       then ds_read_b64_tr_b16 gives V^T in A-operand layout
//   O^T[d][row] = O^T c + V^T P^T   v_mfma_f32_16x16x32, float32 accumulators in registers
// The next tile's K and V loads are issued as soon as this tile's have been read out of their buffers: ~16 KiB in
// flight per wave, 8 waves a CU. Float32 / half query rows over a bfloat16 cache enter the first product as two bfloat16
// numbers (the rounded row and the rounded rest), the softmax weights the second product likewise. The 4 waves'
// (O, m, l) are merged through LDS in a fixed order and written as the split's partial {O[D], m (log2 units), l}; a second kernel merges the splits: out = sum O_s 2^(m_s - M) / sum l_s 2^(m_s - M).
//
// Reference behaviour kept: kernels/llm/qwen35/silo/attn.cpp:100-104,261-290,321-370 (split form, partial layout,
// merge, one launch when the rows' split sizes agree - here: a launch a run of rows whose sizes agree), kernels/llm/museglimmer/silo/attn.cpp:51-55,
// 86-92,120-127 (absolute split positions, ring slots, window), and the rounding model of both (16-bit operands,
// float32 scores, softmax and accumulation; quantized values rounded to half as staged).
#include "ns_internal.hpp"
#include "ns_attn.h"
#include "attn_common.hpp"
#include "attn_host.hpp"
#include "kv_formats.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <mutex>
#include <string>
#include <type_traits>

namespace {

constexpr int WAVES = 4, TILE = 32;
typedef uint32_t u4v __attribute__((ext_vector_type(4)));
typedef uint32_t u4a8 __attribute__((ext_vector_type(4), aligned(8)));   // 16 bytes at an 8-byte aligned address
// Keys and values are read once a pass: their loads carry the non-temporal hint (the cache-policy bit of the direct
// global -> LDS load; __builtin_nontemporal_load elsewhere), which measured ~10 % more HBM bandwidth on streaming reads
constexpr int NT_AUX = 2;

struct DecodeParams {
    const void* q;
    int qt;                     // element type of q: 0 float32, 1 half, 2 bfloat16
    int64_t qs;                 // elements between query rows
    const uint8_t* kc;
    const uint8_t* vc;
    int64_t head_stride, row_stride;   // bytes between key heads / between slots
    int64_t cap;
    int wrap;                   // slots are position % cap (a ring that has wrapped); else slot = position
    int T, Hq, G;
    int causal;                 // 0: every row sees to the pass's last key (the drafter's block)
    int64_t p0, win;
    int64_t kfirst;             // >= 0: every row's first key (a block whose rows all start at one key); else the window's
    int64_t kbs, sp0;           // keys a split, the first split's index (absolute position / kbs)
    int ns;
    int nz;                     // row chunks a (split, key head)
    float sl2;                  // scale x log2(e)
    float* part;                // [T][Hq][ns][D + 2]
    // block-sparse passes (one row a launch): the pass's keys are the listed blocks of 128 laid end to end - key j of
    // the kernel's numbering is key sel[j / 128] * 128 + j % 128 of the cache (-1: no block), and keys past sel_pos
    // are not the row's
    const int32_t* sel;         // [Hkv][selK] block ids of this row, or null
    int selK;
    int selT;                   // rows of a block-list pass (each a row of its own in the kernel's numbering); else 1
    int64_t sel_pos;            // the first row's position
};

template <int D, int KT>
struct TileRegs {
    static constexpr bool DMA = KT == 0 || KT == 3;                      // 16-bit value rows go global -> LDS directly
    static constexpr int KB = D / 32;                                    // k-blocks of 32 features
    static constexpr int KW = DMA ? 4 : 2;                               // words a lane loads per (key tile, k-block)
    static constexpr int CPR = KT == 1 ? D / 16 : KT == 2 ? D / 32 : D / 8;   // 16-byte chunks a value row
    static constexpr int KPI = 64 / CPR;                                 // keys a wave covers per V load
    static constexpr int NLV = TILE / KPI;                               // V loads a lane per tile
    uint32_t k[2][DMA ? 1 : KB][KW];                                     // quantized rows: 8 int8 / 8 nibbles
    uint32_t ksc[2][DMA ? 1 : KB];                                       // a block's half scale (in the low 16 bits)
    uint4 v[DMA ? 1 : NLV];                                              // quantized forms only
    uint32_t vsc[DMA ? 1 : NLV];
};

// QS (bfloat16 rows only): query rows that are not bfloat16 enter the first product as two bfloat16 numbers - the rounded
// value and the rounded rest, 16 significant bits, as the weights enter the second - so a float32 or half row loses
// nothing a half operand would keep (one bfloat16 number a feature cost such rows ~2e-3 of absolute error)
template <int D, int RT, int KT, bool QS = false>
__global__ __launch_bounds__(WAVES * 64, D == 128 ? 2 : 1) void attn_decode_kernel(const DecodeParams p) {
    static_assert(!QS || KT == 3, "query rows in two parts: bfloat16 operands only");
    constexpr bool BF = KT == 3;
    using R = TileRegs<D, KT>;
    constexpr bool DMA = R::DMA;
    constexpr int KB = R::KB, DT = D / 16;
    // a wave's stage: DMA: a key tile and a value tile, unpadded and swizzled, [32][2 D bytes] each; else one padded
    // value tile (rows + 32 bytes)
    constexpr int RS = DMA ? D * 2 : D * 2 + 32;
    constexpr int VTILE = TILE * RS;
    // quantized rows: the tile's raw rows go global -> LDS too, a row as QCH chunks of 16 bytes - the last chunk is the
    // row's last 16 bytes (rows of 136 or 72 bytes are no whole number of chunks: their last chunk overlaps the one before
    // and the scales sit in its upper half) - one buffer a stream behind the value stage
    // (q4_0 rows of 128 values keep the register path: their arithmetic bounds them - 19.7 against 20.7 us for a 4-row
    // pass over 65536 keys - where q8_0 rows gain 13 % and rows of 256 values 11 - 14 %)
    constexpr bool QDMA = KT == 1 || (KT == 2 && D == 256);
    constexpr int QRB = KT == 1 ? D + D / 16 : D / 2 + D / 16;     // bytes a cache row
    constexpr int QVB = KT == 1 ? D : D / 2;                       // of them values
    constexpr int QCH = (QRB + 15) / 16, QROW = QCH * 16, QRAW = TILE * QROW;
    constexpr int QSOFF = (QCH - 1) * 16 + QVB - (QRB - 16);       // where a row's scales sit in its LDS row
    constexpr int QNI = (TILE * QCH + 63) / 64;                    // transfer instructions a tile and stream
    static_assert(!QDMA || (TILE * QCH) % 64 == 32 || (TILE * QCH) % 64 == 0, "the last instruction is whole or half");
    constexpr int STAGE = DMA ? 2 * VTILE : QDMA ? VTILE + 2 * QRAW : VTILE;
    constexpr int OROW = D + 4;                                    // floats a row of a wave's merge buffer
    constexpr int MERGE = RT * 16 * OROW * 4;
    // a wave's own region: its value stage while it streams, its (O, m, l) for the merge afterwards
    constexpr int WREG = ((STAGE > MERGE ? STAGE : MERGE) + 1023) / 1024 * 1024;
    __shared__ __attribute__((aligned(1024))) uint8_t lds[WAVES * WREG];
    __shared__ float ml[WAVES][RT * 16][2];

    const int tid = threadIdx.x, lane = tid & 63, n = lane & 15, g4 = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // the wave's index, known uniform to the compiler
    // (split, key head, row chunk) of this work-group. Work-group ids go round the 8 XCDs, each with its own L2; the row
    // chunks of one (split, head) read the same keys, so they take consecutive ids of ONE XCD and run there together:
    // the keys come from HBM once and from that L2 for the other chunks. With one chunk this is the plain order, splits
    // fastest. The grid is padded to a multiple of 8 (split, head) pairs; the padding leaves at once.
    const int xj = blockIdx.x / 8, u = (xj / p.nz) * 8 + (int) (blockIdx.x % 8), z = xj % p.nz;
    // (a block-list pass holds selT rows with lists of their own: a row is one more factor of the pairs, tr its index)
    const int Hkv = p.Hq / p.G;
    if (u >= p.ns * Hkv * p.selT) return;
    const int split = u % p.ns, hk = (u / p.ns) % Hkv, tr = u / (p.ns * Hkv);
    const int rows = p.T * p.G;
    const int64_t pass_end = p.p0 + p.T;
    const int64_t fmin = p.kfirst >= 0 ? p.kfirst : p.win > 0 ? std::max<int64_t>(0, p.p0 + 1 - p.win) : 0;
    const int64_t jb = std::max((p.sp0 + split) * p.kbs, fmin), je = std::min((p.sp0 + split + 1) * p.kbs, pass_end);

    const uint8_t* kbase = p.kc + (int64_t) hk * p.head_stride;
    const uint8_t* vbase = p.vc + (int64_t) hk * p.head_stride;
    uint8_t* stage = lds + w * WREG;
    const int32_t* selp = p.sel ? p.sel + ((int64_t) tr * Hkv + hk) * p.selK : nullptr;
    const int64_t sel_pos = p.sel_pos + tr;

    // a key's row offset: keys outside [jb, je) are clamped into it (their scores are masked, their values meet P = 0).
    // A wrapped ring's slot is position % cap: the split's first key's slot once, then offsets from it with at most two
    // wraps (a pass's keys span less than two rings). 32-bit arithmetic relative to the split's first key.
    const int64_t jb_slot = p.wrap && jb < je ? jb % p.cap : jb;
    const int span = (int) (je - jb) - 1;
    auto row_off = [&](int rel) __attribute__((always_inline)) -> int64_t {
        const int rc = std::min(std::max(rel, 0), span);
        int64_t slot = jb_slot + rc;
        if (p.wrap) {
            slot = slot >= p.cap ? slot - p.cap : slot;
            slot = slot >= p.cap ? slot - p.cap : slot;
        }
        return slot * p.row_stride;
    };
    // the tile's keys into registers (MFMA A layout) and its values on their way: DMA into LDS buffer `buf`, chunk
    // position cp of key kk holding the row's chunk cp ^ 2 (kk % 8); or raw into registers
    // a listed block's tile: its 32 keys sit together in the cache (a block holds 4 tiles); no block: any valid rows
    auto tile_off = [&](int64_t ti, int j0, int idx) __attribute__((always_inline)) -> int64_t {
        if (!selp) return row_off(j0 + idx);
        const int blk = selp[(ti * TILE) >> 7];
        // (keys of a listed block past the row's position are masked: read the row's own key instead - the cache may end there)
        return std::min<int64_t>((int64_t) (blk < 0 ? 0 : blk) * 128 + ((ti * TILE) & 127) + idx, sel_pos) * p.row_stride;
    };
    // 16-bit rows: a tile's keys (which = 0) or values (1) on their way global -> LDS, 1 KiB a load: position cp of key kk
    // holds the row's 16-byte chunk cp ^ (kk % 16) (keys: the operand reads of 16 keys' same chunk meet no bank
    // conflict) or cp ^ 2 (kk % 8) (values: the transposing reads)
    // (a tile wholly inside the split of an unwrapped, unlisted cache - all but a pass's last - is read at a wave-uniform
    // address plus a 32-bit lane offset: FAST. Rows of 128: the 8 offsets of a stream are worked out once and kept. Rows of
    // 256 - 16 loads a stream, two keys a load - have no registers for that: key kk = kr0 + 2 i is i double-rows on from
    // the tile's base (wave-uniform) plus the lane's own row kr0, and its swizzle splits the same way, since 2 i is even
    // and kr0 one bit: cp ^ (kk % 16) = (cp ^ kr0) ^ (2 i % 16), cp ^ 2 (kk % 8) = (cp ^ 2 kr0) ^ (4 i % 16) - an
    // exclusive-or with a constant and a shift-add a load)
    constexpr bool FAST = DMA;
    constexpr bool FAST_KEPT = DMA && R::NLV <= 8;
    uint32_t koff[FAST_KEPT ? R::NLV : 1], voff[FAST_KEPT ? R::NLV : 1];
    uint32_t lane_row = 0, cpk = 0, cpv = 0;
    if constexpr (FAST_KEPT) {
        const int cp = lane % R::CPR, kr0 = lane / R::CPR;
#pragma unroll
        for (int i = 0; i < R::NLV; ++i) {
            const int kk = kr0 + R::KPI * i;
            koff[i] = (uint32_t) (kk * p.row_stride) + (uint32_t) ((cp ^ (kk & 15)) * 16);
            voff[i] = (uint32_t) (kk * p.row_stride) + (uint32_t) ((cp ^ (2 * (kk & 7))) * 16);
        }
    } else if constexpr (FAST) {
        static_assert(!FAST || FAST_KEPT || R::KPI == 2, "the split of the swizzle assumes two keys a load");
        const uint32_t cp = lane % R::CPR, kr0 = lane / R::CPR;
        lane_row = kr0 * (uint32_t) p.row_stride;
        cpk = cp ^ kr0;
        cpv = cp ^ (2 * kr0);
    }
    // (a pass of several row chunks reads a split's keys once a chunk, the chunks side by side on one XCD: its loads keep
    // the ordinary policy, so that the chunks after the first find the lines in that XCD's L2 - 16 rows x 32 / 8 heads
    // behind 131072 keys 148.5 -> 118.9 us; a pass of one chunk reads every key once and streams)
    const bool stream = p.nz == 1;
    auto to_lds = [&](const uint8_t* src, uint8_t* dst) __attribute__((always_inline)) {
        if (stream) __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*) src, (__attribute__((address_space(3))) void*) dst, 16, 0, NT_AUX);
        else __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*) src, (__attribute__((address_space(3))) void*) dst, 16, 0, 0);
    };
    auto dma_tile = [&](int64_t ti, int which) __attribute__((always_inline)) {
        const int j0 = (int) (ti * TILE - jb);                 // the tile's first key relative to the split's
        if constexpr (FAST) {
            if (!selp && !p.wrap && j0 >= 0 && j0 + TILE - 1 <= span) {
                const uint8_t* base = (which ? vbase : kbase) + (jb_slot + j0) * p.row_stride;
#pragma unroll
                for (int i = 0; i < R::NLV; ++i) {
                    if constexpr (FAST_KEPT) {
                        to_lds(base + (which ? voff[i] : koff[i]), stage + which * VTILE + i * 1024);
                    } else {
                        const uint32_t off = lane_row + ((which ? cpv ^ (uint32_t) ((2 * R::KPI * i) & 14) : cpk ^ (uint32_t) ((R::KPI * i) & 15)) << 4);
                        to_lds(base + (int64_t) (R::KPI * i) * p.row_stride + off, stage + which * VTILE + i * 1024);
                    }
                }
                return;
            }
        }
        const int cp = lane % R::CPR, kr0 = lane / R::CPR;
#pragma unroll
        for (int i = 0; i < R::NLV; ++i) {
            const int kk = kr0 + R::KPI * i;
            const uint8_t* row = (which ? vbase : kbase) + tile_off(ti, j0, kk);
            const int c = which ? cp ^ (2 * (kk & 7)) : cp ^ (kk & 15);
            to_lds(row + c * 16, stage + which * VTILE + i * 1024);
        }
    };
    // quantized rows: the tile's keys (MFMA A layout) and values raw into registers
    // (interior tiles of an unwrapped, unlisted cache: a wave-uniform tile address plus a lane's row offset, worked out once)
    const uint32_t qk_lane = (uint32_t) (n * p.row_stride), qv_lane = (uint32_t) ((lane / R::CPR) * p.row_stride);
    // (soff: where a row's scales start - behind its values in the cache, in its last chunk's upper part in LDS)
    auto load_rows = [&](R& r, auto krow, auto vrow, int soff) __attribute__((always_inline)) {
#pragma unroll
        for (int kt2 = 0; kt2 < 2; ++kt2) {
            const uint8_t* kr = krow(kt2);
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                if constexpr (KT == 1) {
                    // 16 bytes a lane and pair of k-blocks (rows are 8-byte aligned): k-block 2 j + h, lane group g4, slot e
                    // stands for feature 64 j + 16 g4 + 8 h + e - the queries are loaded in the same order - and both
                    // k-blocks of a pair lie in the scale block 2 j + g4 / 2
                    if (kb % 2 == 0) {
                        const u4a8 x = *reinterpret_cast<const u4a8*>(kr + kb * 32 + g4 * 16);
                        r.k[kt2][kb][0] = x[0]; r.k[kt2][kb][1] = x[1];
                        r.k[kt2][kb + 1][0] = x[2]; r.k[kt2][kb + 1][1] = x[3];
                        r.ksc[kt2][kb] = r.ksc[kt2][kb + 1] = *reinterpret_cast<const uint16_t*>(kr + soff + 2 * (kb + g4 / 2));
                    }
                } else {
                    const uint2 x = *reinterpret_cast<const uint2*>(kr + kb * 16 + (g4 & 1) * 8);
                    r.k[kt2][kb][0] = x.x; r.k[kt2][kb][1] = x.y;
                    r.ksc[kt2][kb] = *reinterpret_cast<const uint16_t*>(kr + soff + 2 * kb);
                }
            }
        }
        const int cp = lane % R::CPR;
#pragma unroll
        for (int i = 0; i < R::NLV; ++i) {
            const uint8_t* vr = vrow(i);
            r.v[i] = *reinterpret_cast<const uint4*>(vr + cp * 16);
            if constexpr (KT == 1) r.vsc[i] = *reinterpret_cast<const uint16_t*>(vr + soff + 2 * (cp / 2));
            if constexpr (KT == 2) r.vsc[i] = *reinterpret_cast<const uint16_t*>(vr + soff + 2 * cp);
        }
    };
    auto load_tile = [&](R& r, int64_t ti) __attribute__((always_inline)) {
        const int j0 = (int) (ti * TILE - jb);
        if (!selp && !p.wrap && j0 >= 0 && j0 + TILE - 1 <= span) {
            const uint8_t* kt0 = kbase + (jb_slot + j0) * p.row_stride;
            const uint8_t* vt0 = vbase + (jb_slot + j0) * p.row_stride;
            load_rows(r, [&](int kt2) { return kt0 + kt2 * 16 * p.row_stride + qk_lane; }, [&](int i) { return vt0 + R::KPI * i * p.row_stride + qv_lane; }, QVB);
        } else {
            const int kr0 = lane / R::CPR;
            load_rows(r, [&](int kt2) { return kbase + tile_off(ti, j0, kt2 * 16 + n); }, [&](int i) { return vbase + tile_off(ti, j0, kr0 + R::KPI * i); }, QVB);
        }
    };

    uint32_t qoff5[QDMA ? QNI : 1];
    if constexpr (QDMA) {
#pragma unroll
        for (int i = 0; i < QNI; ++i) {
            const int u = std::min(i * 64 + lane, TILE * QCH - 1), row = u / QCH, c = u % QCH;
            qoff5[i] = (uint32_t) (row * p.row_stride) + (uint32_t) (c < QCH - 1 ? c * 16 : QRB - 16);
        }
    }
    auto qdma_tile = [&](int64_t ti, int which) __attribute__((always_inline)) {
        const int j0 = (int) (ti * TILE - jb);
        const bool plain = !selp && !p.wrap && j0 >= 0 && j0 + TILE - 1 <= span;
        const uint64_t base_v = (uint64_t) (uintptr_t) ((which ? vbase : kbase) + (plain ? (jb_slot + j0) * p.row_stride : 0));
        // (wave-uniform by construction; said so to the compiler, which wants it in scalar registers)
        // (the builtin returns a signed int: each half goes through uint32_t, or a low half with its top bit set would
        // sign-extend over the high one)
        const uint32_t base_lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) base_v);
        const uint32_t base_hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (base_v >> 32));
        const uint8_t* base = reinterpret_cast<const uint8_t*>((uint64_t) base_lo | ((uint64_t) base_hi << 32));
#pragma unroll
        for (int i = 0; i < QNI; ++i) {
            uint32_t off = qoff5[i];
            if (!plain) {
                const int u = std::min(i * 64 + lane, TILE * QCH - 1), row = u / QCH, c = u % QCH;
                off = (uint32_t) tile_off(ti, j0, row) + (uint32_t) (c < QCH - 1 ? c * 16 : QRB - 16);
            }
            if (i < QNI - 1 || (TILE * QCH) % 64 == 0 || lane < 32) {
                const uint32_t m = __builtin_amdgcn_readfirstlane((uint32_t) (uintptr_t) (stage + VTILE + which * QRAW + i * 1024));
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
                // (quantized rows stream whatever the chunks: their passes of several chunks gain nothing from the other policy)
                asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(m), "v"(off), "s"(base) : "memory", "m0");
#pragma clang diagnostic pop
            }
        }
    };
    // the raw tile out of LDS into the register set the quantized path works on (the same registers a global load fills)
    auto qread_tile = [&](R& r) __attribute__((always_inline)) {
        const uint8_t* rk = stage + VTILE;
        const uint8_t* rv = stage + VTILE + QRAW;
        const int kr0 = lane / R::CPR;
        load_rows(r, [&](int kt2) { return rk + (kt2 * 16 + n) * QROW; }, [&](int i) { return rv + (kr0 + R::KPI * i) * QROW; }, QSOFF);
    };

    // ---- this wave's tiles: absolute tile index % 4 == w, over [jb, je). The first one is requested before anything
    // else: nothing in it depends on the queries
    const int64_t tb = jb / TILE, te = jb < je ? (je + TILE - 1) / TILE : tb;
    int64_t ti = tb + ((w - (int) (tb % WAVES) + WAVES) % WAVES);
    R ra, rb;
    if (ti < te) {
        if constexpr (DMA) {
            dma_tile(ti, 0);
            dma_tile(ti, 1);
        } else if constexpr (QDMA) {
            qdma_tile(ti, 0);
            qdma_tile(ti, 1);
        } else {
            load_tile(ra, ti);
        }
    }
    // where this lane reads its key operands in the key tile: key n (and 16 + n), chunk 4 kb + g4 at its swizzled position
    uint32_t k_rd[KB];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) k_rd[kb] = (uint32_t) (uintptr_t) (stage + n * RS + (((kb * 4 + g4) ^ n) * 16));

    // ---- this lane's rows (one per row tile): their key ranges and Q^T operands
    int lo_r[RT], hi_r[RT];     // the row's first and last key in this split, relative to the split's first (none: 1, 0)
    bool live_r[RT];
    s8v qreg[RT][KB], qlo[QS ? RT : 1][KB];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int ri = (z * RT + rt) * 16 + n;
        const bool live = ri < rows;
        const int t = live ? ri / p.G : 0, gq = live ? ri % p.G : 0;
        const int64_t pos = p.p0 + t, first = p.kfirst >= 0 ? p.kfirst : p.win > 0 ? std::max<int64_t>(0, pos + 1 - p.win) : 0;
        live_r[rt] = live;
        // (a row whose last key lies before the split keeps an empty range; the differences fit 32 bits: a split's keys do)
        const int64_t hi64 = std::min(p.causal ? pos : pass_end - 1, je - 1);
        lo_r[rt] = live && hi64 >= jb ? (int) (std::max(first, jb) - jb) : 1;
        hi_r[rt] = live && hi64 >= jb ? (int) (hi64 - jb) : 0;
        // 8 consecutive features per k-block, vector loads all issued before any is used (rows are 16-byte aligned:
        // checked on the host); a dead row reads row 0's and is zeroed
        // feature order of the k-blocks: plain (k-block kb, lane group g4: features 32 kb + 8 g4 ..), q8_0 keys: see load_tile
        auto foff = [&](int kb) { return KT == 1 ? 64 * (kb / 2) + 16 * g4 + 8 * (kb % 2) : 32 * kb + 8 * g4; };
        const int64_t qoff = (int64_t) (t + tr) * p.qs + ((int64_t) hk * p.G + gq) * D;
        if (p.qt == 0) {
            float4 raw[KB][2];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                raw[kb][0] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.q) + qoff + foff(kb));
                raw[kb][1] = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.q) + qoff + foff(kb) + 4);
            }
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                const float f[8] = {raw[kb][0].x, raw[kb][0].y, raw[kb][0].z, raw[kb][0].w, raw[kb][1].x, raw[kb][1].y, raw[kb][1].z, raw[kb][1].w};
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const short hi = to16<BF>(f[i]);
                    qreg[rt][kb][i] = live ? hi : (short) 0;
                    if constexpr (QS) qlo[rt][kb][i] = live ? to16<true>(f[i] - bf16_to_f32((uint16_t) hi)) : (short) 0;
                }
            }
        } else {
            uint4 raw[KB];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) raw[kb] = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.q) + qoff + foff(kb));
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                const uint32_t ww[4] = {raw[kb].x, raw[kb].y, raw[kb].z, raw[kb].w};
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint16_t b16 = (uint16_t) (ww[i >> 1] >> (16 * (i & 1)));
                    // the same 16-bit type as the kernel's operands passes through; the other is converted
                    const short v = (p.qt == 2) == BF ? (short) b16 : to16<BF>(p.qt == 1 ? f16_to_f32(b16) : bf16_to_f32(b16));
                    qreg[rt][kb][i] = live ? v : (short) 0;
                    if constexpr (QS) qlo[rt][kb][i] = live && p.qt == 1 ? to16<true>(f16_to_f32(b16) - bf16_to_f32((uint16_t) v)) : (short) 0;
                }
            }
        }
    }

    float m_r[RT], l_r[RT];
    f4v o[RT][DT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        m_r[rt] = -INFINITY;
        l_r[rt] = 0.0f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[rt][dt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
    }

    // 16-bit rows: loads complete in the order they were issued - ... K(i), V(i), K(i + 1), V(i + 1) ... - so a wait
    // that leaves one tile's NLV loads outstanding has seen everything older. MORE: the wave has a tile after this one
    // (at ti + WAVES), whose keys are requested as soon as this tile's have been read out of the key buffer and whose
    // values as soon as this tile's have been read out of the value buffer.
    auto process_tile = [&](R& r, int64_t ti, auto more_c) __attribute__((always_inline)) {
        constexpr bool more = decltype(more_c)::value;
        const int64_t j0 = ti * TILE;
        if constexpr (!DMA) {
            // ---- the value tile dequantized into this wave's LDS stage, [key][D] halfs
            const int c = lane % R::CPR, kr0 = lane / R::CPR;
#pragma unroll
            for (int i = 0; i < R::NLV; ++i) {
                uint8_t* dst = stage + (kr0 + R::KPI * i) * RS;
                const _Float16 d = __builtin_bit_cast(_Float16, (uint16_t) r.vsc[i]);
                if constexpr (KT == 1) {
                    *reinterpret_cast<s8v*>(dst + c * 32) = dq8x8(r.v[i].x, r.v[i].y, d);
                    *reinterpret_cast<s8v*>(dst + c * 32 + 16) = dq8x8(r.v[i].z, r.v[i].w, d);
                } else {
                    // values 0 .. 15: the low nibbles of the 16 bytes, 16 .. 31: the high ones
                    *reinterpret_cast<s8v*>(dst + c * 64) = dq4x8(r.v[i].x, r.v[i].y, 0, d);
                    *reinterpret_cast<s8v*>(dst + c * 64 + 16) = dq4x8(r.v[i].z, r.v[i].w, 0, d);
                    *reinterpret_cast<s8v*>(dst + c * 64 + 32) = dq4x8(r.v[i].x, r.v[i].y, 4, d);
                    *reinterpret_cast<s8v*>(dst + c * 64 + 48) = dq4x8(r.v[i].z, r.v[i].w, 4, d);
                }
            }
        }
        // ---- S^T = K Q^T for both 16-key tiles and every row tile. 16-bit rows: the key operands come out of the key
        // buffer - both 16-key halves at once at D = 128, a half at a time at D = 256 (32 registers instead of 64) - and
        // the next tile's keys are requested as soon as the last of them has been read
        f4v s[RT][2];
        if constexpr (DMA) {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(R::NLV) : "memory");           // V(i) may be out; K(i) is in
            constexpr int KH = D == 128 ? 2 : 1;
#pragma unroll
            for (int h0 = 0; h0 < 2; h0 += KH) {
                s8v kall[KH][KB];
#pragma unroll
                for (int kt2 = 0; kt2 < KH; ++kt2)
#pragma unroll
                    for (int kb = 0; kb < KB; ++kb)
                        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(kall[kt2][kb]) : "v"(k_rd[kb]), "n"((h0 + kt2) * 16 * RS));
                // (every register the reads fill is named, so that no use of one moves above the wait)
#pragma unroll
                for (int kt2 = 0; kt2 < KH; ++kt2) {
                    if constexpr (KB == 4)
                        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(kall[kt2][0]), "+v"(kall[kt2][1]), "+v"(kall[kt2][2]), "+v"(kall[kt2][3])::"memory");
                    else
                        asm volatile("s_waitcnt lgkmcnt(0)"
                                     : "+v"(kall[kt2][0]), "+v"(kall[kt2][1]), "+v"(kall[kt2][2]), "+v"(kall[kt2][3]), "+v"(kall[kt2][4]),
                                       "+v"(kall[kt2][5]), "+v"(kall[kt2][6]), "+v"(kall[kt2][7])::"memory");
                }
                if constexpr (more) {
                    if (h0 + KH == 2) dma_tile(ti + WAVES, 0);
                }
#pragma unroll
                for (int kt2 = 0; kt2 < KH; ++kt2)
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) {
                        f4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                        for (int kb = 0; kb < KB; ++kb) {
                            acc = mfma16<BF>(kall[kt2][kb], qreg[rt][kb], acc);
                            if constexpr (QS) acc = mfma16<BF>(kall[kt2][kb], qlo[rt][kb], acc);
                        }
                        s[rt][h0 + kt2] = acc;
                    }
            }
        } else {
#pragma unroll
            for (int kt2 = 0; kt2 < 2; ++kt2) {
                s8v ka[KB];
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) {
                    const _Float16 d = __builtin_bit_cast(_Float16, (uint16_t) r.ksc[kt2][kb]);
                    if constexpr (KT == 1) {
                        ka[kb] = dq8x8(r.k[kt2][kb][0], r.k[kt2][kb][1], d);
                    } else {
                        ka[kb] = dq4x8(r.k[kt2][kb][0], r.k[kt2][kb][1], g4 >= 2 ? 4 : 0, d);
                    }
                }
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    f4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int kb = 0; kb < KB; ++kb) acc = mfma16<BF>(ka[kb], qreg[rt][kb], acc);
                    s[rt][kt2] = acc;
                }
            }
        }
        // ---- online softmax a row (this lane: row n of each row tile, keys j0 + 16 kt2 + 4 g4 + i)
        // a row's keys inside this tile: lo .. lo + span of 0 .. 31 (none: lo = 64 puts every key below it), in 32-bit
        // arithmetic relative to the split's first key. Tiles that no live row's edge crosses - all but the first and last
        // of a pass - take no comparison at all (a wave-uniform branch)
        const int j0r = (int) (j0 - jb);
        int hi_tile = INT32_MAX;
        if (selp) {
            // (a listed block's keys count up to the row's own position; a hole in the list has none)
            const int blk = selp[j0 >> 7];
            hi_tile = blk < 0 ? j0r - 1 : (int) ((j0 & ~(int64_t) 127) - jb + std::min<int64_t>(127, sel_pos - (int64_t) blk * 128));
        }
        int lo_t[RT];
        unsigned span_t[RT];
        bool edge = false;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const int lo_ = std::min(std::max(lo_r[rt] - j0r, 0), 32);
            const int hi = std::min(std::max(std::min(hi_r[rt], hi_tile) - j0r, -1), 31);
            lo_t[rt] = hi < lo_ ? 64 : lo_;
            span_t[rt] = hi < lo_ ? 0u : (unsigned) (hi - lo_);
            edge |= live_r[rt] && (lo_ > 0 || hi < 31);                   // (a dead row may keep its zero scores)
        }
        float x[RT][8];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
            for (int e = 0; e < 8; ++e) x[rt][e] = s[rt][e >> 2][e & 3];
        if (__any(edge)) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    x[rt][e] = (unsigned) ((e >> 2) * 16 + g4 * 4 + (e & 3) - lo_t[rt]) <= span_t[rt] ? x[rt][e] : -INFINITY;
        }
        // the scale rides in the exponent's fused multiply-add: weights 2^(x sl2 - m), m the running maximum of x sl2
        // (0 in its place while a row has seen no key: its weights are 2^(-inf) = 0 either way)
        // (a bfloat16 cache: the weights enter the second product as two bfloat16 numbers, the rounded weight and the rounded
        // rest - 16 significant bits between them, where one alone would carry 8 and cost the output ~1.6e-3 of relative L2)
        s8v pb[RT], pl[BF ? RT : 1];
        float cs[RT];
        bool shrink = false;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            const float mx = rows_max(fmaxf(fmaxf(fmaxf(x[rt][0], x[rt][1]), fmaxf(x[rt][2], x[rt][3])), fmaxf(fmaxf(x[rt][4], x[rt][5]), fmaxf(x[rt][6], x[rt][7]))));
            const float mn = fmaxf(m_r[rt], mx * p.sl2);
            const float ms = mn == -INFINITY ? 0.0f : mn;
            cs[rt] = fast_exp2(m_r[rt] - ms);
            shrink |= m_r[rt] != mn;
            float sum = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float pv = fast_exp2(fmaf(x[rt][e], p.sl2, -ms));
                sum += pv;
                pb[rt][e] = to16<BF>(pv);
                if constexpr (BF) pl[rt][e] = to16<BF>(pv - __builtin_bit_cast(float, (uint32_t) (uint16_t) pb[rt][e] << 16));
            }
            m_r[rt] = mn;
            l_r[rt] = l_r[rt] * cs[rt] + rows_sum(sum);
        }
        // the running output shrinks only when some row's maximum moved (rare once a pass is under way): wave-uniform
        if (__any(shrink)) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) o[rt][dt] *= cs[rt];
        }
        // ---- O^T += V^T P^T: the value tile read back transposed. The reads and their waits are written in assembly:
        // the compiler's own tracking of LDS writes by DMA would wait for EVERY outstanding load here (the next tile's
        // too) before any LDS read it can see. DMA: this tile's loads are older than the next tile's 2 KB + NLV
        // (issued after them, in order), so waiting until only those remain makes the tile visible
        if constexpr (DMA) {
            if constexpr (more) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(R::NLV) : "memory");     // K(i + 1) may be out
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        } else {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
        const int kk = g4 * 4 + (n >> 2);                      // the key row this lane's address names (and + 16)
        constexpr int HALF = D == 128 ? DT / 2 : DT / 4;       // column tiles whose reads are in flight together
#pragma unroll
        for (int h2 = 0; h2 < DT / HALF; ++h2) {
            s4v lo[HALF], hi[HALF];
#pragma unroll
            for (int d2 = 0; d2 < HALF; ++d2) {
                const int dt = h2 * HALF + d2;
                uint32_t src;
                if constexpr (DMA) {
                    const int c = (dt * 2 + ((n & 3) >> 1)) ^ (2 * (kk & 7));
                    src = (uint32_t) (uintptr_t) (stage + VTILE + kk * RS + c * 16 + (n & 1) * 8);
                } else {
                    src = (uint32_t) (uintptr_t) (stage + kk * RS + (dt * 16 + 4 * (n & 3)) * 2);
                }
                asm volatile("ds_read_b64_tr_b16 %0, %2\n\tds_read_b64_tr_b16 %1, %2 offset:%3" : "=&v"(lo[d2]), "=&v"(hi[d2]) : "v"(src), "n"(16 * RS));
            }
#pragma unroll
            for (int d2 = 0; d2 < HALF; ++d2) {
                const int dt = h2 * HALF + d2;
                // reads return in order: 2 (HALF - 1 - d2) may still be out when this pair is needed
                asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(lo[d2]), "+v"(hi[d2]) : "n"(2 * (HALF - 1 - d2)));
                const s8v va = {lo[d2][0], lo[d2][1], lo[d2][2], lo[d2][3], hi[d2][0], hi[d2][1], hi[d2][2], hi[d2][3]};
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) {
                    o[rt][dt] = mfma16<BF>(va, pb[rt], o[rt][dt]);
                    if constexpr (BF) o[rt][dt] = mfma16<BF>(va, pl[rt], o[rt][dt]);
                }
            }
        }
        // every read of the stage has returned: it is free for the next loads
        asm volatile("" ::: "memory");
        if constexpr (DMA && more) dma_tile(ti + WAVES, 1);
    };

    // ---- the wave's tiles. Quantized rows alternate two register sets, the next tile's loads issued before this one's math
    if (ti < te) {
        const std::true_type more;
        const std::false_type last;
        if constexpr (DMA) {
            for (; ti + WAVES < te; ti += WAVES) process_tile(ra, ti, more);
            process_tile(ra, ti, last);
        } else if constexpr (QDMA) {
            // the tile's raw rows have landed (requested a tile ago); once they are in registers the next tile's are
            // requested into the same two buffers and travel under this tile's arithmetic
            for (;; ti += WAVES) {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                qread_tile(ra);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                const bool has_next = ti + WAVES < te;
                if (has_next) {
                    qdma_tile(ti + WAVES, 0);
                    qdma_tile(ti + WAVES, 1);
                }
                process_tile(ra, ti, more);
                if (!has_next) break;
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        } else {
            while (ti + 2 * WAVES < te) {
                load_tile(rb, ti + WAVES);
                process_tile(ra, ti, more);
                load_tile(ra, ti + 2 * WAVES);
                process_tile(rb, ti + WAVES, more);
                ti += 2 * WAVES;
            }
            if (ti + WAVES < te) {
                load_tile(rb, ti + WAVES);
                process_tile(ra, ti, more);
                process_tile(rb, ti + WAVES, last);
            } else {
                process_tile(ra, ti, last);
            }
        }
    }

    // ---- the 4 waves' (O, m, l) merged in wave order and written as the split's partial. Each wave parks its live rows
    // in its own region (free: every read of its stage has returned), one barrier, then a thread a (row, 4 features)
    const int live_rows = std::min(RT * 16, rows - z * RT * 16);
    float* ow = reinterpret_cast<float*>(stage);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (rt * 16 + n < live_rows) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) *reinterpret_cast<f4v*>(ow + (rt * 16 + n) * OROW + dt * 16 + g4 * 4) = o[rt][dt];
            if (g4 == 0) {
                ml[w][rt * 16 + n][0] = m_r[rt];
                ml[w][rt * 16 + n][1] = l_r[rt];
            }
        }
    }
    __syncthreads();
    for (int idx = tid; idx < live_rows * (D / 4); idx += WAVES * 64) {
        const int row = idx / (D / 4), c = idx % (D / 4), ri = z * RT * 16 + row;
        const int t = ri / p.G, gq = ri % p.G;
        float M = -INFINITY;
#pragma unroll
        for (int k = 0; k < WAVES; ++k) M = fmaxf(M, ml[k][row][0]);
        float L = 0.0f;
        f4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int k = 0; k < WAVES; ++k) {
            const float f = ml[k][row][0] == -INFINITY ? 0.0f : fast_exp2(ml[k][row][0] - M);
            L += ml[k][row][1] * f;
            const f4v ok = *reinterpret_cast<const f4v*>(reinterpret_cast<const float*>(lds + k * WREG) + row * OROW + c * 4);
            acc = k == 0 ? ok * f : acc + ok * f;
        }
        // partial rows are D + 2 floats: 8-byte aligned
        float* pr = p.part + (((int64_t) (t + tr) * p.Hq + hk * p.G + gq) * p.ns + split) * (D + 2);
        *reinterpret_cast<float2*>(pr + c * 4) = float2{acc[0], acc[1]};
        *reinterpret_cast<float2*>(pr + c * 4 + 2) = float2{acc[2], acc[3]};
        if (c == 0) *reinterpret_cast<float2*>(pr + D) = float2{M, L};
    }
}

// The splits of a (row, head) merged by a work-group of 4 waves: out = sum_s O_s w_s / sum_s l_s w_s, w_s = 2^(m_s - M).
// Wave k adds the splits s = k, k + 4, ... in ascending order (fused multiply-adds; a lane owns D / 64 features in 8-byte
// pieces) and the four sums are added as (0 + 1) + (2 + 3): a fixed shape, so the result does not depend on how many
// empty splits a pass appends to a row's own (their weight is 0). Every wave works out all the weights itself (no
// barrier before the sums), and its first 32 splits' values are requested before the weights exist.
// (MERGE_W waves: 4, or 8 for passes over one or two key heads, whose rows have 256 partials and more - chosen by the heads,
// never by the rows or the splits of a pass, so a row is summed in the same shape whatever pass it is in: 8 / 1 heads over
// 131072 keys, merge 6.1 -> 4.6 us)
constexpr int MERGE_MAX_NS = 2048;

template <int D, int MERGE_W>
__global__ __launch_bounds__(MERGE_W * 64) void attn_merge_kernel(const float* __restrict__ part, int ns, int qt, void* __restrict__ out) {
    constexpr int C = D / 128, PS = D + 2, PF = 32, B = 16;
    __shared__ float wsh[MERGE_W][MERGE_MAX_NS + MERGE_W * PF];
    __shared__ float2 sums[MERGE_W][C][64];
    const int lane = threadIdx.x & 63, k = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t rh = blockIdx.x;
    const float* pr = part + rh * ns * PS;
    // (slots past the last split are not fetched - a wave-uniform test a slot; they enter with weight 0 either way, and a
    // step of few splits - 32 a head behind 4096 keys - would spend most of its time fetching them again and again:
    // heads of 256, 8 waves: 6.3 -> 3.8 us, the same bits)
    float2 x[PF][C];
#pragma unroll
    for (int j = 0; j < PF; ++j) {
        if (k + MERGE_W * j < ns) {
#pragma unroll
            for (int c = 0; c < C; ++c) x[j][c] = *reinterpret_cast<const float2*>(pr + (int64_t) (k + MERGE_W * j) * PS + 2 * (lane + 64 * c));
        } else {
#pragma unroll
            for (int c = 0; c < C; ++c) x[j][c] = float2{0.0f, 0.0f};
        }
    }
    float mx = -INFINITY;
    for (int s = lane; s < ns; s += 64) mx = fmaxf(mx, pr[(int64_t) s * PS + D]);
    mx = wave_max(mx);
    // this wave's splits: nk of them, walked in batches of B after the first PF (slots past the last hold weight 0)
    const int nk = ns > k ? (ns - k + MERGE_W - 1) / MERGE_W : 0;
    const int njp = std::max(PF, (nk + B - 1) / B * B), nsz = MERGE_W * njp;
    float* wk = wsh[k];
    float ls = 0.0f;
    for (int s = lane; s < nsz; s += 64) {
        float wgt = 0.0f;
        if (s < ns) {
            const float2 mlv = *reinterpret_cast<const float2*>(pr + (int64_t) s * PS + D);
            wgt = mlv.x == -INFINITY ? 0.0f : fast_exp2(mlv.x - mx);
            ls = fmaf(mlv.y, wgt, ls);
        }
        wk[s] = wgt;
    }
    ls = wave_sum(ls);
    // wk was written by this wave's own lanes: a wave's LDS operations complete in order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    float2 acc[C];
#pragma unroll
    for (int c = 0; c < C; ++c) acc[c] = float2{0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < PF; ++j) {
        const float wgt = wk[k + MERGE_W * j];
#pragma unroll
        for (int c = 0; c < C; ++c) {
            acc[c].x = fmaf(x[j][c].x, wgt, acc[c].x);
            acc[c].y = fmaf(x[j][c].y, wgt, acc[c].y);
        }
    }
    for (int j0 = PF; j0 < njp; j0 += B) {
        float2 y[B][C];
#pragma unroll
        for (int j = 0; j < B; ++j) {
            if (k + MERGE_W * (j0 + j) < ns) {
#pragma unroll
                for (int c = 0; c < C; ++c) y[j][c] = *reinterpret_cast<const float2*>(pr + (int64_t) (k + MERGE_W * (j0 + j)) * PS + 2 * (lane + 64 * c));
            } else {
#pragma unroll
                for (int c = 0; c < C; ++c) y[j][c] = float2{0.0f, 0.0f};
            }
        }
#pragma unroll
        for (int j = 0; j < B; ++j) {
            const float wgt = wk[k + MERGE_W * (j0 + j)];
#pragma unroll
            for (int c = 0; c < C; ++c) {
                acc[c].x = fmaf(y[j][c].x, wgt, acc[c].x);
                acc[c].y = fmaf(y[j][c].y, wgt, acc[c].y);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < C; ++c) sums[k][c][lane] = acc[c];
    __syncthreads();
    if (k != 0) return;
#pragma unroll
    for (int c = 0; c < C; ++c) {
        const float2 s0 = sums[0][c][lane], s1 = sums[1][c][lane], s2 = sums[2][c][lane], s3 = sums[3][c][lane];
        float ax = (s0.x + s1.x) + (s2.x + s3.x), ay = (s0.y + s1.y) + (s2.y + s3.y);
        if constexpr (MERGE_W == 8) {
            const float2 s4 = sums[4][c][lane], s5 = sums[5][c][lane], s6 = sums[6][c][lane], s7 = sums[7][c][lane];
            ax += (s4.x + s5.x) + (s6.x + s7.x);
            ay += (s4.y + s5.y) + (s6.y + s7.y);
        }
        const float a = ls > 0.0f ? ax / ls : 0.0f, b = ls > 0.0f ? ay / ls : 0.0f;
        const int64_t i = rh * D + 2 * (lane + 64 * c);
        if (qt == 0) *reinterpret_cast<float2*>(reinterpret_cast<float*>(out) + i) = float2{a, b};
        else if (qt == 1) *reinterpret_cast<uint32_t*>(reinterpret_cast<uint16_t*>(out) + i) = (uint32_t) (uint16_t) to16<false>(a) | (uint32_t) (uint16_t) to16<false>(b) << 16;
        else *reinterpret_cast<uint32_t*>(reinterpret_cast<uint16_t*>(out) + i) = (uint32_t) (uint16_t) to16<true>(a) | (uint32_t) (uint16_t) to16<true>(b) << 16;
    }
}

// The same merge for passes of many rows and few splits - a prompt pass cut into key splits leaves tens of thousands of
// (row, head) pairs of 2 - 64 partials each, and a work-group a pair is then mostly launch: 16 lanes a pair, 16 pairs a
// work-group, a lane D / 16 features as 8-byte pieces (a partial of D + 2 floats is 8-byte aligned), the splits in ascending
// order with fused multiply-adds. out = sum O_s 2^(m_s - M) / sum l_s 2^(m_s - M), 0 where the row saw no key.
template <int D>
__global__ __launch_bounds__(256) void attn_merge_rows_kernel(const float* __restrict__ part, int ns, int qt, int64_t rows, void* __restrict__ out) {
    constexpr int PS = D + 2, NP = D / 32;                       // 8-byte pieces a lane
    const int64_t rh = (int64_t) blockIdx.x * 16 + (threadIdx.x >> 4);
    if (rh >= rows) return;
    const int li = threadIdx.x & 15;
    const float* pr = part + rh * ns * PS;
    float mx = -INFINITY;
    for (int s = 0; s < ns; ++s) mx = fmaxf(mx, pr[(int64_t) s * PS + D]);
    float2 acc[NP];
#pragma unroll
    for (int j = 0; j < NP; ++j) acc[j] = float2{0.0f, 0.0f};
    float ls = 0.0f;
    for (int s = 0; s < ns; ++s) {
        const float* ps = pr + (int64_t) s * PS;
        float2 x[NP];
#pragma unroll
        for (int j = 0; j < NP; ++j) x[j] = *reinterpret_cast<const float2*>(ps + 2 * (li + 16 * j));
        const float2 mlv = *reinterpret_cast<const float2*>(ps + D);
        const float wgt = mlv.x == -INFINITY ? 0.0f : fast_exp2(mlv.x - mx);
        ls = fmaf(mlv.y, wgt, ls);
#pragma unroll
        for (int j = 0; j < NP; ++j) {
            acc[j].x = fmaf(x[j].x, wgt, acc[j].x);
            acc[j].y = fmaf(x[j].y, wgt, acc[j].y);
        }
    }
#pragma unroll
    for (int j = 0; j < NP; ++j) {
        const float a = ls > 0.0f ? acc[j].x / ls : 0.0f, b = ls > 0.0f ? acc[j].y / ls : 0.0f;
        const int64_t i = rh * D + 2 * (li + 16 * j);
        if (qt == 0) *reinterpret_cast<float2*>(reinterpret_cast<float*>(out) + i) = float2{a, b};
        else if (qt == 1) *reinterpret_cast<uint32_t*>(reinterpret_cast<uint16_t*>(out) + i) = (uint32_t) (uint16_t) to16<false>(a) | (uint32_t) (uint16_t) to16<false>(b) << 16;
        else *reinterpret_cast<uint32_t*>(reinterpret_cast<uint16_t*>(out) + i) = (uint32_t) (uint16_t) to16<true>(a) | (uint32_t) (uint16_t) to16<true>(b) << 16;
    }
}

// ---- host side ----------------------------------------------------------------------------------------------------

// work-groups the key splits aim for (key heads x splits): two a CU at head size 128, one at 256 (its LDS footprint admits
// one a CU; 256 against 512 measured 17.6 against 23.2 us at 32K keys, and half the partials to merge). A split's partial
// is written and read again for every query row on it - T x G rows of D + 2 floats against the split's 2 kbs rows of
// keys and values - so 16-bit caches whose key heads serve 8 or more query heads take half as many, twice as long
// splits (G = 8, 64K keys, 4 rows: 30.9 -> 29.7 us; G = 16, 4 rows: 44.7 -> 40.5; one row: within 0.5 us either way);
// quantized rows keep the two work-groups a CU their arithmetic needs (128K keys of q8_0: 35.0 against 37.8 us) - but
// for one or two key heads, whose 256 or 512 partials a query head cost the merge more than that (8 / 1 heads over
// 131072 q8_0 keys: 21.9 -> 18.7 us, 16 / 2 heads 23.7 -> 22.3).
// The rule may depend on the heads and the cache form, never on the rows of a pass. NS_DEC_WGS overrides (tuning)
int64_t target_wgs(int64_t D, int64_t G, int kt, int64_t Hkv) {
    const int64_t v = ns_tune_get(NS_TUNE_DEC_WGS);
    return v > 0 ? v : D == 256 || (G >= 8 && (kt == 0 || kt == 3)) || (kt == 1 && Hkv <= 2) ? 256 : 512;
}
// keys a split for a row that sees `keys` keys: a multiple of 128 (4 waves x 32-key tiles)
// (quantized rows whose rule aims for 512 work-groups: short contexts take 256 of splits up to 384 or 512 keys first - a split's
// fixed cost and its partial weigh more than the second work-group a CU gains; 64 / 4 heads over 16383 q8_0 keys: one row
// 13.8 -> 12.5 us, four rows 28.2 -> 20.7. 16-bit rows gained in one layout of the caches and lost in another: unchanged)
int64_t dec_kbs(int64_t keys, int64_t Hkv, int64_t D, int64_t G, int kt) {
    const int64_t t = target_wgs(D, G, kt, Hkv), want = (keys * Hkv + t - 1) / t;
    const int64_t kbs = std::max<int64_t>(128, (want + 127) / 128 * 128);
    if (t != 512 || ns_tune_get(NS_TUNE_DEC_WGS) > 0 || kt == 0 || kt == 3) return kbs;
    const int64_t want2 = (keys * Hkv + 255) / 256, kbs2 = std::max<int64_t>(128, (want2 + 127) / 128 * 128);
    // (up to 512 keys a split where a key head serves 8 query heads and more - their partials weigh most - else 384: 32 / 8
    // heads over 12500 q8_0 keys in 256 splits of 512 keys 14.7 us, in 392 of 256 keys 13.9)
    return kbs2 <= (G >= 8 ? 512 : 384) ? kbs2 : kbs;
}
inline int64_t row_first(int64_t pos, int64_t win) { return win > 0 ? std::max<int64_t>(0, pos - win + 1) : 0; }

// the pass's T x G rows of a key head ride in row tiles of 16: one tile up to 16 rows, else chunks of two tiles (more
// rows than 32 re-read the keys once per chunk)
template <int D, int KT>
int launch_rt(ns_gpu* g, const DecodeParams& p, int rows, dim3 grid_xy) {
    // (quantized rows of 256 as two row tiles take the whole register file - 512 with a few spilled - and still beat two
    // chunks that each lift and widen the tile: 24 / 4 heads x 4 rows behind 131072 q8_0 keys 110.8 -> 76.4 us, q4_0 106.4 -> 72.7)
    // (rows of 256 in two bfloat16 parts stay one row tile a chunk: two tiles of them would spill a fifth of the kernel's registers)
    const bool parts = KT == 3 && p.qt != 2;
    const int RT = rows <= 16 || (parts && D == 256) ? 1 : 2;
    DecodeParams c = p;
    c.nz = (rows + RT * 16 - 1) / (RT * 16);
    const int64_t pairs = (int64_t) grid_xy.x * grid_xy.y, wgs = (pairs + 7) / 8 * 8 * c.nz;
    if (wgs >= (int64_t) 1 << 31) return ns_fail("ns_attn_decode: too many work-groups");
    const dim3 grid((unsigned) wgs);
    if constexpr (KT == 3) {
        if (parts) {
            if (RT == 1) attn_decode_kernel<D, 1, KT, true><<<grid, WAVES * 64, 0, g->q>>>(c);
            else if constexpr (D == 128) attn_decode_kernel<D, 2, KT, true><<<grid, WAVES * 64, 0, g->q>>>(c);
            NS_LAUNCHED("attn_decode");
            return 0;
        }
    }
    if (RT == 1) attn_decode_kernel<D, 1, KT><<<grid, WAVES * 64, 0, g->q>>>(c);
    else attn_decode_kernel<D, 2, KT><<<grid, WAVES * 64, 0, g->q>>>(c);
    NS_LAUNCHED("attn_decode");
    return 0;
}

template <int D>
int launch_kt(ns_gpu* g, int kt, const DecodeParams& p, int rows, dim3 grid_xy) {
    switch (kt) {
        case 0: return launch_rt<D, 0>(g, p, rows, grid_xy);
        case 1: return launch_rt<D, 1>(g, p, rows, grid_xy);
        case 2: return launch_rt<D, 2>(g, p, rows, grid_xy);
        default: return launch_rt<D, 3>(g, p, rows, grid_xy);
    }
}

template <int D>
int launch_merge(ns_gpu* g, const float* part, int ns, int qt, int64_t rh, void* out, bool wide = false) {
    if (ns > MERGE_MAX_NS) return ns_fail("ns_attn_decode: more key splits than the merge holds");
    if (wide) attn_merge_kernel<D, 8><<<(unsigned) rh, 8 * 64, 0, g->q>>>(part, ns, qt, out);
    else attn_merge_kernel<D, 4><<<(unsigned) rh, 4 * 64, 0, g->q>>>(part, ns, qt, out);
    NS_LAUNCHED("attn_merge");
    return 0;
}

template <int D, int QT>
int decode_typed(ns_gpu* g, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv,
                 int64_t cap, int64_t p0, int64_t win, const DecodeExtra& x, float scale, void* out, float* scratch) {
    const int64_t rb = kv_row_bytes(kt, D);
    const int esz = QT == 0 ? 4 : 2;
    const int causal = x.causal;
    DecodeParams p{};
    p.selT = 1;
    p.qt = QT;
    p.kc = (const uint8_t*) kc;
    p.vc = (const uint8_t*) vc;
    p.head_stride = pm ? rb : cap * rb;
    p.row_stride = pm ? Hkv * rb : rb;
    p.cap = cap;
    p.wrap = !pm && p0 + T > cap;
    p.Hq = (int) Hq;
    p.G = (int) (Hq / Hkv);
    p.causal = causal;
    p.win = win;
    p.kfirst = x.kfirst;
    p.sl2 = (scale > 0.0f ? scale : 1.0f / sqrtf((float) D)) * 1.4426950408889634f;
    const int64_t last = p0 + T - 1;
    auto first_of = [&](int64_t r) { return x.kfirst >= 0 ? x.kfirst : row_first(p0 + r, win); };
    auto kb_of = [&](int64_t r) { return dec_kbs(p0 + r + 1 - first_of(r), Hkv, D, Hq / Hkv, kt); };
    // A causal pass is one launch when its rows' own split sizes agree (a row's bits must not depend on the rows that
    // share its pass). Where they do not - the pass straddles a key count at which the split size steps - the reference
    // launches a row at a time (kernels/llm/qwen35/silo/attn.cpp:344-350); here each run of consecutive rows with one
    // split size is a launch: every row is still cut by its own split size, and a pass has two runs, not T launches
    // (8 rows across the step at 65536 keys: 212 -> 58 us). A pass that is not causal is always one launch, cut by its
    // first row's key count (the longest: every row ends at the pass's last key) - kernels/llm/museglimmer/silo/attn.cpp:282-291
    const int64_t nsa = (x.scratch_floats > 0 ? x.scratch_floats : ns_attn_decode_scratch(T, Hq, Hkv, D, p0, win)) / (T * Hq * (D + 2));
    auto launch = [&](int64_t r0, int64_t nr, int64_t kb) -> int {
        const int64_t pp = p0 + r0, sp0 = first_of(r0) / kb, ns = (pp + nr - 1) / kb - sp0 + 1;
        if (ns > nsa) return ns_fail("ns_attn_decode: more key splits than the scratch holds");
        DecodeParams c = p;
        c.q = (const uint8_t*) q + r0 * qs * esz;
        c.qs = qs;
        c.T = (int) nr;
        c.p0 = pp;
        c.kbs = kb;
        c.sp0 = sp0;
        c.ns = (int) ns;
        c.part = scratch + r0 * Hq * nsa * (D + 2);
        if (x.marks && ns_profile_mark(g, 0)) return -1;
        if (launch_kt<D>(g, kt, c, (int) (nr * c.G), dim3((unsigned) ns, (unsigned) Hkv))) return -1;
        if (x.marks && ns_profile_mark(g, 1)) return -1;
        if (launch_merge<D>(g, c.part, (int) ns, QT, nr * Hq, (uint8_t*) out + r0 * Hq * D * esz, Hkv <= 2)) return -1;
        return x.marks ? ns_profile_mark(g, 2) : 0;
    };
    if (!causal) return launch(0, T, dec_kbs(last + 1 - first_of(0), Hkv, D, Hq / Hkv, kt));
    for (int64_t r = 0; r < T;) {
        const int64_t kb = kb_of(r);
        int64_t r1 = r + 1;
        while (r1 < T && kb_of(r1) == kb) ++r1;
        if (launch(r, r1 - r, kb)) return -1;
        r = r1;
    }
    return 0;
}

int decode_checked(ns_gpu* g, const char* who, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T,
                   int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, const DecodeExtra& x, float scale, void* out,
                   float* scratch) {
    NS_TRY
    const std::string w(who);
    if (T <= 0) return 0;
    if (T > 16) return ns_fail(w + ": 1..16 rows (a decode or verify pass)");
    if (D != 128 && D != 256) return ns_fail(w + ": heads of 128 or 256");
    if (Hkv <= 0 || Hq <= 0 || Hq % Hkv) return ns_fail(w + ": query heads a multiple of the key heads");
    if (kt < 0 || kt > 3) return ns_fail(w + ": a cache form 0 (half), 1 (q8_0), 2 (q4_0) or 3 (bfloat16)");
    if (qt < 0 || qt > 2) return ns_fail(w + ": rows of type 0 (float32), 1 (half) or 2 (bfloat16)");
    if (p0 < 0 || cap <= 0 || win < 0) return ns_fail(w + ": a position, a capacity and a window of 0 or more");
    if (x.kfirst > p0) return ns_fail(w + ": a block's first key lies at or before its first row");
    if (Hkv > 65535) return ns_fail(w + ": at most 65535 key heads");
    const int64_t need = pm ? p0 + T : (win > 0 ? std::min(p0 + T, win + T - 1) : p0 + T);
    if (need > cap) return ns_fail(w + (win > 0 ? ": the cache's ring is shorter than the window and the pass" : ": past the cache's capacity"));
    if (!scratch) return ns_fail(w + ": no scratch");
    if ((uintptr_t) scratch % 8) return ns_fail(w + ": scratch 8-byte aligned");
    if (!q || !kc || !vc || !out) return ns_fail(w + ": a null buffer");
    if ((uintptr_t) q % 16 || qs % (qt == 0 ? 4 : 8)) return ns_fail(w + ": query rows 16-byte aligned");
    if (((uintptr_t) kc | (uintptr_t) vc) % 16 && (kt == 0 || kt == 3)) return ns_fail(w + ": caches 16-byte aligned");
    if (((uintptr_t) kc | (uintptr_t) vc) % 8) return ns_fail(w + ": caches 8-byte aligned");
    NS_HIP(hipSetDevice(g->dev));
#define NS_DISPATCH(DD, QQ) return decode_typed<DD, QQ>(g, kt, pm, q, qs, kc, vc, T, Hq, Hkv, cap, p0, win, x, scale, out, scratch)
    if (D == 128) {
        if (qt == 0) NS_DISPATCH(128, 0);
        if (qt == 1) NS_DISPATCH(128, 1);
        NS_DISPATCH(128, 2);
    } else {
        if (qt == 0) NS_DISPATCH(256, 0);
        if (qt == 1) NS_DISPATCH(256, 1);
        NS_DISPATCH(256, 2);
    }
#undef NS_DISPATCH
    NS_CATCH
}

}  // namespace

// Block-sparse decode over a position-major half cache [pos][Hkv][128] (MiniMax-M3: kernels/llm/minimaxm3/mm3.cpp:118-190
// with sel != NULL): row t attends the K blocks of 128 keys sel[(t Hkv + hk) K ..] names (-1: none), cut at its own
// position. Rows choose their own blocks, so a row is a launch (split over its K x 128 listed keys) and a merge.
int ns_attn_decode_sel(ns_gpu* g, const char* who, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K,
                       float* out, int64_t T, int64_t Hq, int64_t Hkv, int64_t pos0, float scale, float* scratch, size_t scratch_floats) {
    NS_TRY
    constexpr int D = 128;
    const std::string w(who);
    if (T <= 0) return 0;
    if (Hkv <= 0 || Hq <= 0 || Hq % Hkv) return ns_fail(w + ": query heads a multiple of the key heads");
    if (K < 0 || K > (int64_t) 1 << 20) return ns_fail(w + ": a block count");
    if (!q || !kc || !vc || !out || !sel || !scratch) return ns_fail(w + ": a null buffer");
    if ((uintptr_t) q % 16 || ((uintptr_t) kc | (uintptr_t) vc) % 16) return ns_fail(w + ": rows 16-byte aligned");
    NS_HIP(hipSetDevice(g->dev));
    if (K == 0) return ns_fill(g, out, 0, (size_t) (T * Hq * D) * sizeof(float));     // nothing listed: zeros (l = 0)
    // A (row, key head) with its own list is a unit of the launch. A decode or verify pass (up to 16 rows) cuts a row's
    // listed keys by the row's own count, whatever rows share the pass (a row's bits do not depend on them). A prompt
    // pass has units enough: its rows' keys are cut only while rows x key heads leave the chip short of work-groups -
    // from 128 rows on not at all - and the rows go as many to a launch as the scratch holds partials for (a launch a row,
    // the first form: 2048 rows x 64 / 4 heads with 16 blocks each 34.8 ms)
    const int64_t keys = K * 128;
    int64_t kbs = dec_kbs(keys, Hkv, D, Hq / Hkv, 0);
    if (T > DECODE_ROWS) {
        const int64_t want = std::max<int64_t>(1, std::min((keys + kbs - 1) / kbs, (512 + T * Hkv - 1) / (T * Hkv)));
        kbs = ((keys + want - 1) / want + 127) / 128 * 128;
    }
    const int64_t ns = (keys + kbs - 1) / kbs;
    if ((size_t) (Hq * ns * (D + 2)) > scratch_floats) return ns_fail(w + ": the pass needs more scratch than the library keeps");
    const int64_t rows_a_launch = std::min<int64_t>({T, (int64_t) (scratch_floats / (size_t) (Hq * ns * (D + 2))), 65535 / Hkv});
    if (rows_a_launch < 1) return ns_fail(w + ": too many key heads");
    DecodeParams p{};
    p.qt = 0;
    p.qs = Hq * D;
    p.kc = (const uint8_t*) kc;
    p.vc = (const uint8_t*) vc;
    p.head_stride = 2 * D;
    p.row_stride = Hkv * 2 * D;
    p.cap = keys;
    p.wrap = 0;
    p.T = 1;
    p.Hq = (int) Hq;
    p.G = (int) (Hq / Hkv);
    p.causal = 1;
    p.kfirst = -1;
    p.p0 = keys - 1;            // in the kernel's numbering the row sees every listed key; sel_pos cuts the real ones
    p.win = 0;
    p.kbs = kbs;
    p.sp0 = 0;
    p.ns = (int) ns;
    p.sl2 = scale * 1.4426950408889634f;
    p.part = scratch;
    p.selK = (int) K;
    p.selT = 1;
    for (int64_t t0 = 0; t0 < T; t0 += rows_a_launch) {
        const int64_t nr = std::min(rows_a_launch, T - t0);
        p.q = q + t0 * Hq * D;
        p.sel = sel + t0 * Hkv * K;
        p.sel_pos = pos0 + t0;
        p.selT = (int) nr;
        if (launch_kt<D>(g, 0, p, p.G, dim3((unsigned) ns, (unsigned) (Hkv * nr)))) return -1;
        // (a verify pass's rows are merged as a decode pass's are; a prompt's many rows of few partials 16 pairs a work-group)
        if (T <= DECODE_ROWS ? launch_merge<D>(g, scratch, (int) ns, 0, nr * Hq, out + t0 * Hq * D)
                             : ns_attn_merge_partials(g, D, scratch, ns, 0, nr * Hq, out + t0 * Hq * D))
            return -1;
    }
    return 0;
    NS_CATCH
}

// the merge of [rows][ns][D + 2] partials for the prompt kernel's key splits (the same kernel, the same layout)
int ns_attn_merge_partials(ns_gpu* g, int64_t D, const float* part, int64_t ns, int qt, int64_t rows, void* out) {
    if (ns > MERGE_MAX_NS) return ns_fail("ns_attn_prompt: more key splits than the merge holds");
    // (a prompt pass: many (row, head) pairs of few partials each - 16 pairs a work-group, each walking its partials one
    // after the other: up to 8 of them, or up to 16 where the pairs fill the chip; a work-group a pair otherwise - 17 rows x
    // 32 heads of 32 partials: 50.6 -> 34.1 us the pass, 256 rows of 16: 127 against 150. The choice depends on the
    // pass's shape alone, so a pass is always merged the same way)
    if (ns <= 8 || (ns <= 16 && rows >= 2048)) {
        const unsigned wgs = (unsigned) ((rows + 15) / 16);
        if (D == 128) attn_merge_rows_kernel<128><<<wgs, 256, 0, g->q>>>(part, (int) ns, qt, rows, out);
        else attn_merge_rows_kernel<256><<<wgs, 256, 0, g->q>>>(part, (int) ns, qt, rows, out);
        NS_LAUNCHED("attn_merge_rows");
        return 0;
    }
    return D == 128 ? launch_merge<128>(g, part, (int) ns, qt, rows, out) : launch_merge<256>(g, part, (int) ns, qt, rows, out);
}

// used by the exact-API routing in attn_api.cpp
int ns_attn_decode_any(ns_gpu* g, const char* who, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T,
                       int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, const DecodeExtra& x, float scale, void* out,
                       float* scratch) {
    return decode_checked(g, who, qt, kt, pm, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, win, x, scale, out, scratch);
}

// ---- a decode entry point that allocates nothing ---------------------------------------------------------------------
// Callers under HIP graph capture, tight serving loops and harnesses that forbid allocation cannot hand over a scratch
// buffer they would have to hipMalloc first. ns_attn_decode_static is ns_attn_decode_t with the partials in an array that
// is part of the library's code object: each GPU the library runs on holds its own copy, at its own address, until the
// process ends. In host code the array's name is only a handle for hipGetSymbolAddress - never a device address - so
// the address is looked up once a device (ns_gpu_open calls ns_attn_static_scratch_init with the device current) and
// every launch is given that pointer. Nothing in it has to start at zero: a pass writes every partial it later merges.
// Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two ns_gpu of one device, or two streams)
// race.
static __device__ __align__(256) float ns_static_scratch[NS_ATTN_STATIC_SCRATCH_FLOATS];

namespace {
constexpr int STATIC_MAX_DEVS = 64;
float* static_scratch_ptr[STATIC_MAX_DEVS] = {};
std::mutex static_scratch_mu;
}  // namespace

int ns_attn_static_scratch_init(int dev) {
    if (dev < 0 || dev >= STATIC_MAX_DEVS) return ns_fail("ns_attn_decode_static: device index past the table");
    std::lock_guard<std::mutex> lock(static_scratch_mu);
    if (static_scratch_ptr[dev]) return 0;
    void* ptr = nullptr;
    NS_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(ns_static_scratch)));
    if (!ptr) return ns_fail("ns_attn_decode_static: the scratch array has no address on this device");
    static_scratch_ptr[dev] = (float*) ptr;
    return 0;
}

extern "C" {

int ns_attn_decode_static(ns_gpu* g, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq,
                          int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, float scale, void* out) {
    if (T <= 0) return 0;
    if (!g || g->dev < 0 || g->dev >= STATIC_MAX_DEVS || !static_scratch_ptr[g->dev]) return ns_fail("ns_attn_decode_static: the device's scratch array was not set up");
    if (T > 16 || Hq <= 0 || Hkv <= 0 || (D != 128 && D != 256)) return ns_fail("ns_attn_decode_static: 1..16 rows, heads of 128 or 256");
    const int64_t need = ns_attn_decode_scratch(T, Hq, Hkv, D, p0, win);
    if (need > (int64_t) NS_ATTN_STATIC_SCRATCH_FLOATS)
        return ns_fail("ns_attn_decode_static: the pass needs " + std::to_string(need) + " floats of scratch, the array holds " +
                       std::to_string((int64_t) NS_ATTN_STATIC_SCRATCH_FLOATS) + " (use ns_attn_decode_t with a buffer of the caller's)");
    DecodeExtra x;
    x.marks = false;                                   // (the profiling events are created on first use: an allocation)
    return decode_checked(g, "ns_attn_decode_static", qt, kt, pm, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, win, x, scale, out, static_scratch_ptr[g->dev]);
}

int64_t ns_attn_decode_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0, int64_t win) {
    if (T <= 0 || Hq <= 0 || Hkv <= 0) return 0;
    int64_t ns = 1;
    // (the cache form is not an argument: the count holds for the 16-bit rule, q8_0's and q4_0's)
    for (int kt = 0; kt < 3; ++kt) {
        auto kbs = [&](int64_t keys) { return dec_kbs(keys, Hkv, D, Hq / Hkv, kt); };
        // a run of rows launched on its own: the row's own split size over its own first key to the pass's last
        // the pass in one launch: from its first row's first key to its last row's last; causal or not, the last row's
        // key count bounds every row's
        const int64_t f0 = row_first(p0, win), last = p0 + T - 1;
        for (int64_t r = 0; r < T; ++r) {
            const int64_t pos = p0 + r, first = row_first(pos, win), kb = kbs(last + 1 - first), kb2 = kbs(pos + 1 - first);
            ns = std::max(ns, pos / kb2 - first / kb2 + 1);
            ns = std::max(ns, last / kb - f0 / kb + 1);
            ns = std::max(ns, last / kb2 - f0 / kb2 + 1);
        }
    }
    return T * Hq * ns * (D + 2);
}

int ns_attn_decode_t(ns_gpu* g, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq,
                     int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, float scale, void* out, float* scratch) {
    return decode_checked(g, "ns_attn_decode_t", qt, kt, pm, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, win, DecodeExtra{}, scale, out, scratch);
}

int ns_q35_attn_decode_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D) {
    return T >= 1 && T <= 16 && (D == 128 || D == 256) && Hkv > 0 && Hq > 0 && Hq % Hkv == 0;
}
int64_t ns_q35_attn_decode_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0) { return ns_attn_decode_scratch(T, Hq, Hkv, D, p0, 0); }
int ns_q35_attn_decode(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D,
                       int64_t cap, int64_t p0, float* out, float* scratch) {
    return decode_checked(g, "ns_q35_attn_decode", 0, 0, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, DecodeExtra{}, 0.0f, out, scratch);
}
int ns_q35_attn_decode_kv(ns_gpu* g, int kt, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv,
                          int64_t D, int64_t cap, int64_t p0, float* out, float* scratch) {
    if (kt < 0 || kt > 2) return ns_fail("ns_q35_attn_decode_kv: a cache form 0 (half), 1 (q8_0) or 2 (q4_0)");
    return decode_checked(g, "ns_q35_attn_decode_kv", 0, kt, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, DecodeExtra{}, 0.0f, out, scratch);
}

int ns_nhs_attn_decode_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D) { return ns_q35_attn_decode_supported(T, Hq, Hkv, D); }
int64_t ns_nhs_attn_decode_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0) { return ns_attn_decode_scratch(T, Hq, Hkv, D, p0, 0); }
int ns_nhs_attn_decode(ns_gpu* g, const float* q, int64_t qs, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D,
                       int64_t cap, int64_t p0, float* out, float* scratch) {
    return decode_checked(g, "ns_nhs_attn_decode", 0, 0, 0, q, qs, kc, vc, T, Hq, Hkv, D, cap, p0, 0, DecodeExtra{}, 0.0f, out, scratch);
}

int ns_mg_attn_decode_supported(int64_t T, int64_t Hq, int64_t Hkv, int64_t D) { return ns_q35_attn_decode_supported(T, Hq, Hkv, D); }
int64_t ns_mg_attn_decode_scratch(int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t p0, int64_t win) {
    return ns_attn_decode_scratch(T, Hq, Hkv, D, p0, win);
}
int ns_mg_attn_decode(ns_gpu* g, const float* q, const void* kc, const void* vc, int64_t T, int64_t Hq, int64_t Hkv, int64_t D, int64_t cap,
                      int64_t p0, int64_t win, float* out, float* scratch) {
    return decode_checked(g, "ns_mg_attn_decode", 0, 0, 0, q, Hq * D, kc, vc, T, Hq, Hkv, D, cap, p0, win, DecodeExtra{}, 0.0f, out, scratch);
}

}  // extern "C"
