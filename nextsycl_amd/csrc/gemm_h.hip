// gemm_h.hip: the half products of the engines' MLA prompt chain - ns_to_f16, ns_gemm_f16, ns_gemm_batch_h - and its gather of
// half cache rows, ns_gather_h, for gfx950.
//
// The reference hands these to oneMKL (kernels/llm/glm5next/glm.cpp:208-276); an engine's prompt branch calls them around
// its masked softmax (llm/deepseek2/src/engine.rs:1170-1244). The fused route through ns_mla_decode_latent is the fast
// one here; these exist so that the branch binds and runs unchanged: y [T, N] (+)= x [T, K] . op(w), half operands,
// float32 sums on v_mfma_f32_16x16x32_f16, any T / N / K / strides.
//
// Work split: a work-group of 4 waves a 64 x 64 block of y (a wave 32 x 32: 2 x 2 tiles), K in steps of 32. Rows of x - and of
// w where op(w) = w^T, w [N, K] - are K-contiguous, which is the MFMA operand's own packing: a lane's 8 values are one
// 16-byte load, no LDS. Where op(w) = w, w [K, N], a step's 32 x 64 block of w goes through LDS and comes back transposed
// (ds_read_b64_tr_b16). Rows and columns past the edge are clamped on the way in and not written; a K that is no multiple of
// 8, or operands that are not 16-byte aligned, take the loads element by element.
//
// Products large enough to fill the chip (a prompt chunk's scores and weighted sums: tens of thousands of rows) take the
// tiled form instead: 256 x 128 of y a work-group of 8 waves (a wave 64 x 64: 4 x 4 tiles, two waves a SIMD), K in stages
// of 64 that travel global -> LDS directly (global_load_lds_dwordx4), two stages ahead into three buffers, one barrier a
// stage; the 16-byte chunks of a row are XOR-swizzled on the global side so that the operand reads (ds_read_b128 of 16
// rows' same chunk; the transposing read where op(w) = w) meet no bank conflict. 87 flop a byte staged.
#include "ns_internal.hpp"
#include "ns_mla.h"
#include "attn_common.hpp"
#include "kv_formats.hpp"

#include <algorithm>

namespace {

typedef uint32_t u4v __attribute__((ext_vector_type(4)));

struct GemmParams {
    const uint16_t* x;
    const uint16_t* w;
    float* y;
    int64_t T, N, K, ldx, sx, ldw, sw, ldy, sy;
    int accumulate, vec_x, vec_w;
};

// 8 consecutive halfs of a row from element k on, zeros from K on
__device__ __forceinline__ s8v load8(const uint16_t* row, int64_t k, int64_t K, bool vec) {
    if (vec && k + 8 <= K) return __builtin_bit_cast(s8v, *reinterpret_cast<const u4v*>(row + k));
    s8v r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = k + e < K ? (short) row[k + e] : (short) 0;
    return r;
}

__device__ __forceinline__ s4v load4(const uint16_t* row, int64_t k, int64_t K, bool vec) {
    if (vec && k + 4 <= K) return *reinterpret_cast<const s4v*>(row + k);
    s4v r;
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = k + e < K ? (short) row[k + e] : (short) 0;
    return r;
}

template <bool TRANS_W>
__global__ __launch_bounds__(256) void gemm_h_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) uint16_t wt[32][64 + 8];      // op(w) = w: a step's block of w, rows padded by 16 bytes
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 15, g4 = lane >> 4, wv = tid >> 6;
    const int64_t b = blockIdx.z, r0 = (int64_t) blockIdx.y * 64 + (wv >> 1) * 32, c0 = (int64_t) blockIdx.x * 64 + (wv & 1) * 32;
    const uint16_t* x = p.x + b * p.sx;
    const uint16_t* w = p.w + b * p.sw;
    float* y = p.y + b * p.sy;
    f4v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
    // the lane's rows of x (and of w^T): tile i's row n, clamped into the matrix
    const uint16_t* xr[2];
    const uint16_t* wr[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        xr[i] = x + std::min<int64_t>(r0 + 16 * i + n, p.T - 1) * p.ldx;
        wr[i] = w + (TRANS_W ? std::min<int64_t>(c0 + 16 * i + n, p.N - 1) * p.ldw : 0);
    }
    for (int64_t k0 = 0; k0 < p.K; k0 += 32) {
        s8v a[2], bb[2];
        if constexpr (TRANS_W) {
#pragma unroll
            for (int i = 0; i < 2; ++i) a[i] = load8(xr[i], k0 + 8 * g4, p.K, p.vec_x);
#pragma unroll
            for (int j = 0; j < 2; ++j) bb[j] = load8(wr[j], k0 + 8 * g4, p.K, p.vec_w);
        } else {
            // the block w[k0 .. k0 + 31][64 columns of this work-group] into LDS: 256 threads, 8 columns each
            __syncthreads();
            {
                const int kr = tid >> 3, cc = (tid & 7) * 8;
                const int64_t kk = k0 + kr, col = (int64_t) blockIdx.x * 64 + cc;
                s8v v;
                if (kk < p.K && p.vec_w && col + 8 <= p.N) {
                    v = __builtin_bit_cast(s8v, *reinterpret_cast<const u4v*>(w + kk * p.ldw + col));
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] = kk < p.K && col + e < p.N ? (short) w[kk * p.ldw + col + e] : (short) 0;
                }
                *reinterpret_cast<s8v*>(&wt[kr][cc]) = v;
            }
            __syncthreads();
            // lane i of a 16-lane group receives rows k .. k + 3 of column c + i: the lane names row 4 g4 + n / 4 (and 16 more),
            // columns c + 4 (n % 4) ..
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int cb = (wv & 1) * 32 + 16 * j + 4 * (n & 3);
                const s4v lo = lds_read_tr16(&wt[4 * g4 + (n >> 2)][cb]);
                const s4v hi = lds_read_tr16(&wt[16 + 4 * g4 + (n >> 2)][cb]);
                bb[j] = s8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
            // (the operand's k-slots are then rows 4 g4 .. + 3 and 16 + 4 g4 .. + 3 of the step: x is read in the same order)
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const s4v lo = load4(xr[i], k0 + 4 * g4, p.K, p.vec_x), hi = load4(xr[i], k0 + 16 + 4 * g4, p.K, p.vec_x);
                a[i] = s8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            }
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = mfma16<false>(a[i], bb[j], acc[i][j]);
    }
    // a lane holds rows 4 g4 .. + 3 of column n of each tile
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int64_t col = c0 + 16 * j + n;
            if (col >= p.N) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t row = r0 + 16 * i + 4 * g4 + e;
                if (row >= p.T) continue;
                float* d = y + row * p.ldy + col;
                *d = p.accumulate ? *d + acc[i][j][e] : acc[i][j][e];
            }
        }
}

// ---- the tiled form
constexpr int TN = 128, TK = 64, TWAVES = 8;

// TM: rows of y a work-group (256; 128 where x has too few rows for that: a wave then 32 x 64)
template <bool TRANS_W, int TM>
__global__ __launch_bounds__(TWAVES * 64, 1) void gemm_h_tiled_kernel(const GemmParams p) {
    constexpr int TA_BYTES = TM * TK * 2, TB_BYTES = TN * TK * 2, TSTAGE = TA_BYTES + TB_BYTES;      // 32 (16) KiB + 16 KiB
    constexpr int TDMA_A = TA_BYTES / 1024 / TWAVES, TDMA_B = TB_BYTES / 1024 / TWAVES;             // transfers a wave and stage: 4 (2) + 2
    constexpr int RW = TM / 4, IT = RW / 16;                                                        // rows a wave, its row tiles
    __shared__ __attribute__((aligned(1024))) uint8_t lds[3 * TSTAGE];
    typedef __attribute__((address_space(3))) uint8_t lds_u8;
    lds_u8* const L = (lds_u8*) lds;
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 15, g4 = lane >> 4;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6), wm = w >> 1, wn = w & 1;
    const int64_t b = blockIdx.z, r0 = (int64_t) blockIdx.y * TM, c0 = (int64_t) blockIdx.x * TN;
    const uint8_t* const xb = reinterpret_cast<const uint8_t*>(p.x + b * p.sx);
    const uint8_t* const wb = reinterpret_cast<const uint8_t*>(p.w + b * p.sw);
    float* const y = p.y + b * p.sy;

    // ---- a stage's transfers. x rows (and w rows where op(w) = w^T) are 128 bytes of the stage = 8 chunks: unit 8 r + pos of the
    // buffer holds chunk pos ^ ((r / 2) % 8) of row r; rows past the edge are clamped to the last (never written).
    // op(w) = w: a stage holds 64 k-rows of 128 columns = 16 chunks: unit 16 k + pos holds chunk pos ^ 2 (k % 8); chunks past the
    // last column are clamped to the last whole one.
    uint32_t offa[TDMA_A], offb[TDMA_B];
#pragma unroll
    for (int j = 0; j < TDMA_A; ++j) {
        const int u = (w * TDMA_A + j) * 64 + lane, r = u >> 3, kc = (u & 7) ^ ((r >> 1) & 7);
        offa[j] = (uint32_t) ((std::min<int64_t>(r0 + r, p.T - 1) - r0) * p.ldx * 2 + kc * 16);
    }
#pragma unroll
    for (int j = 0; j < TDMA_B; ++j) {
        const int u = (w * TDMA_B + j) * 64 + lane;
        if constexpr (TRANS_W) {
            const int r = u >> 3, kc = (u & 7) ^ ((r >> 1) & 7);
            offb[j] = (uint32_t) ((std::min<int64_t>(c0 + r, p.N - 1) - c0) * p.ldw * 2 + kc * 16);
        } else {
            const int k = u >> 4, c = (u & 15) ^ (2 * (k & 7));
            offb[j] = (uint32_t) ((int64_t) k * p.ldw * 2 + (std::min<int64_t>(c0 + 8 * c, p.N - 8) - c0) * 2);
        }
    }
    auto dma16 = [&](const uint8_t* base_, uint32_t off, lds_u8* dst) __attribute__((always_inline)) {
        const uint32_t m = __builtin_amdgcn_readfirstlane((uint32_t) (uintptr_t) dst);
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"                   // (m0 is reserved: nothing of the compiler's lives in it across this)
        asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m), "v"(off), "s"(base_) : "memory", "m0");
#pragma clang diagnostic pop
    };
    auto dma = [&](int stage, int64_t kt) __attribute__((always_inline)) {
        lds_u8* const sa = L + stage * TSTAGE;
        lds_u8* const sb = sa + TA_BYTES;
        // (lane offsets are relative to the block's first row / column: they stay within 32 bits whatever the matrix)
        const uint8_t* const xa = xb + (r0 * p.ldx + kt * TK) * 2;
        const uint8_t* const wa = TRANS_W ? wb + (c0 * p.ldw + kt * TK) * 2 : wb + (kt * TK * p.ldw + c0) * 2;
#pragma unroll
        for (int j = 0; j < TDMA_A; ++j) dma16(xa, offa[j], sa + (w * TDMA_A + j) * 1024);
#pragma unroll
        for (int j = 0; j < TDMA_B; ++j) dma16(wa, offb[j], sb + (w * TDMA_B + j) * 1024);
    };

    // ---- this lane's operand addresses within a stage: x rows wm 64 + 16 i + n, chunk 4 kk + g4 (swizzle (n / 2) % 8: the rows'
    // other terms are multiples of 16); w^T rows likewise; w: rows 32 kk + 8 g4 + n / 4 (+ 4), columns wn 64 + 16 j + 4 (n % 4)
    const uint32_t a_rd = (uint32_t) ((wm * RW + n) * 128), swz = (uint32_t) ((n >> 1) & 7);
    const uint32_t b_rd = (uint32_t) (TA_BYTES + (wn * 64 + n) * 128);
    const uint32_t bt_rd = (uint32_t) (TA_BYTES + (8 * g4 + (n >> 2)) * 256 + (n & 1) * 8);

    f4v acc[IT][4];
#pragma unroll
    for (int i = 0; i < IT; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f4v{0.0f, 0.0f, 0.0f, 0.0f};

    const int64_t nk = p.K / TK;
    dma(0, 0);
    if (nk > 1) dma(1, 1);
    int stage = 0;
    for (int64_t kt = 0; kt < nk; ++kt) {
        // this wave's transfers of stage kt have landed when at most stage kt + 1's are still out, and its reads of the stage
        // about to be refilled have returned; the barrier makes both everybody's
        if (kt + 1 < nk) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(TDMA_A + TDMA_B) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (kt + 2 < nk) dma(stage >= 1 ? stage - 1 : 2, kt + 2);
        lds_u8* const S = L + stage * TSTAGE;
#pragma unroll
        for (int kk = 0; kk < TK / 32; ++kk) {
            s8v a[IT], bb[4];
#pragma unroll
            for (int i = 0; i < IT; ++i)
                a[i] = *reinterpret_cast<const __attribute__((address_space(3))) s8v*>(S + a_rd + i * 16 * 128 + (((uint32_t) (kk * 4 + g4) ^ swz) << 4));
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (TRANS_W) {
                    bb[j] = *reinterpret_cast<const __attribute__((address_space(3))) s8v*>(S + b_rd + j * 16 * 128 + (((uint32_t) (kk * 4 + g4) ^ swz) << 4));
                } else {
                    const uint32_t c = (uint32_t) (wn * 8 + 2 * j + ((n & 3) >> 1));
                    const uint32_t sl = (uint32_t) (2 * (n >> 2));
                    const s4v lo = lds_read_tr16((void*) (S + bt_rd + kk * 32 * 256 + ((c ^ sl) << 4)));
                    const s4v hi = lds_read_tr16((void*) (S + bt_rd + kk * 32 * 256 + 4 * 256 + ((c ^ (sl + 8)) << 4)));
                    bb[j] = s8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                }
            }
#pragma unroll
            for (int i = 0; i < IT; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = mfma16<false>(a[i], bb[j], acc[i][j]);
        }
        stage = stage == 2 ? 0 : stage + 1;
    }
#pragma unroll
    for (int i = 0; i < IT; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t col = c0 + wn * 64 + 16 * j + n;
            if (col >= p.N) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t row = r0 + wm * RW + 16 * i + 4 * g4 + e;
                if (row >= p.T) continue;
                float* d = y + row * p.ldy + col;
                *d = p.accumulate ? *d + acc[i][j][e] : acc[i][j][e];
            }
        }
}

__global__ __launch_bounds__(256) void to_f16_kernel(const float* __restrict__ x, uint16_t* __restrict__ y, int64_t n) {
    const int64_t i = ((int64_t) blockIdx.x * 256 + threadIdx.x) * 4;
    if (i + 4 <= n && ((uintptr_t) x % 16 == 0) && ((uintptr_t) y % 8 == 0)) {
        const float4 v = *reinterpret_cast<const float4*>(x + i);
        typedef uint16_t us4v __attribute__((ext_vector_type(4)));
        *reinterpret_cast<us4v*>(y + i) = us4v{f32_to_f16(v.x), f32_to_f16(v.y), f32_to_f16(v.z), f32_to_f16(v.w)};
    } else {
        for (int64_t j = i; j < n && j < i + 4; ++j) y[j] = f32_to_f16(x[j]);
    }
}

// out [n][C] = the rows idx[i] of src, 16 bytes a thread
__global__ __launch_bounds__(256) void gather_h_kernel(const u4v* __restrict__ src, const int32_t* __restrict__ idx, u4v* __restrict__ out, int64_t n, int cv) {
    const int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (i >= n * cv) return;
    const int64_t r = i / cv, c = i - r * cv;
    out[i] = src[(int64_t) idx[r] * cv + c];
}

int gemm_h(ns_gpu* g, const char* who, int64_t batch, int trans_w, int64_t T, int64_t N, int64_t K, const uint16_t* x, int64_t ldx, int64_t sx,
           const uint16_t* w, int64_t ldw, int64_t sw, float* y, int64_t ldy, int64_t sy, int accumulate) {
    const std::string s(who);
    if (batch <= 0 || T <= 0 || N <= 0) return 0;
    if (K < 0 || ldx < K || ldy < N || ldw < (trans_w ? K : N)) return ns_fail(s + ": rows at least as far apart as they are long");
    if (!g || !x || !w || !y) return ns_fail(s + ": a null buffer");
    if (batch > 65535 || (T + 63) / 64 > 65535) return ns_fail(s + ": at most 65535 products and 4194240 rows a call");
    NS_HIP(hipSetDevice(g->dev));
    GemmParams p{x, w, y, T, N, K, ldx, sx, ldw, sw, ldy, sy, accumulate, 0, 0};
    p.vec_x = (uintptr_t) x % 16 == 0 && ldx % 8 == 0 && sx % 8 == 0;
    p.vec_w = (uintptr_t) w % 16 == 0 && ldw % 8 == 0 && sw % 8 == 0;
    // the tiled form: aligned operands, whole stages of K, enough of y to be worth 256 x 128 blocks, lane offsets within 32 bits
    // (256-row blocks from 192 rows on, 128-row blocks from 64: a batch of a row's heads against its cells is 64 - 128 rows a product)
    const bool tiled = p.vec_x && p.vec_w && K > 0 && K % TK == 0 && T >= 64 && N >= 64 && (trans_w || N % 8 == 0) && ldx < ((int64_t) 1 << 22) &&
                       ldw < ((int64_t) 1 << 22);
    if (tiled) {
        const int64_t tm = T >= 192 ? 256 : 128;
        const dim3 grid((unsigned) ((N + TN - 1) / TN), (unsigned) ((T + tm - 1) / tm), (unsigned) batch);
        if (tm == 256) {
            if (trans_w) gemm_h_tiled_kernel<true, 256><<<grid, TWAVES * 64, 0, g->q>>>(p);
            else gemm_h_tiled_kernel<false, 256><<<grid, TWAVES * 64, 0, g->q>>>(p);
        } else {
            if (trans_w) gemm_h_tiled_kernel<true, 128><<<grid, TWAVES * 64, 0, g->q>>>(p);
            else gemm_h_tiled_kernel<false, 128><<<grid, TWAVES * 64, 0, g->q>>>(p);
        }
        NS_LAUNCHED("gemm_h_tiled");
        return 0;
    }
    const dim3 grid((unsigned) ((N + 63) / 64), (unsigned) ((T + 63) / 64), (unsigned) batch);
    if (trans_w) gemm_h_kernel<true><<<grid, 256, 0, g->q>>>(p);
    else gemm_h_kernel<false><<<grid, 256, 0, g->q>>>(p);
    NS_LAUNCHED("gemm_h");
    return 0;
}

}  // namespace

extern "C" {

int ns_to_f16(ns_gpu* g, const float* x, uint16_t* y, int64_t n) {
    NS_TRY
    if (n <= 0) return 0;
    if (!g || !x || !y) return ns_fail("ns_to_f16: a null buffer");
    NS_HIP(hipSetDevice(g->dev));
    to_f16_kernel<<<(unsigned) ((n + 1023) / 1024), 256, 0, g->q>>>(x, y, n);
    NS_LAUNCHED("to_f16");
    return 0;
    NS_CATCH
}

int ns_gather_h(ns_gpu* g, const uint16_t* src, const int32_t* idx, uint16_t* out, int64_t n, int64_t C) {
    NS_TRY
    if (n <= 0 || C <= 0) return 0;
    if (C % 8 != 0) return ns_fail("ns_gather_h: row width not a multiple of 8");
    if (!g || !src || !idx || !out) return ns_fail("ns_gather_h: a null buffer");
    if ((uintptr_t) src % 16 || (uintptr_t) out % 16) return ns_fail("ns_gather_h: rows 16-byte aligned");
    if ((n * (C / 8) + 255) / 256 >= (int64_t) 1 << 31) return ns_fail("ns_gather_h: too many rows");
    NS_HIP(hipSetDevice(g->dev));
    gather_h_kernel<<<(unsigned) ((n * (C / 8) + 255) / 256), 256, 0, g->q>>>(reinterpret_cast<const u4v*>(src), idx, reinterpret_cast<u4v*>(out), n, (int) (C / 8));
    NS_LAUNCHED("gather_h");
    return 0;
    NS_CATCH
}

int ns_gemm_f16(ns_gpu* g, int64_t T, int64_t N, int64_t K, const uint16_t* x, int64_t ldx, const uint16_t* w, float* y, int64_t ldy, int accumulate) {
    NS_TRY
    return gemm_h(g, "ns_gemm_f16", 1, 1, T, N, K, x, ldx, 0, w, K, 0, y, ldy, 0, accumulate);
    NS_CATCH
}

int ns_gemm_batch_h(ns_gpu* g, int64_t batch, int trans_w, int64_t T, int64_t N, int64_t K, const uint16_t* x, int64_t ldx, int64_t sx,
                    const uint16_t* w, int64_t ldw, int64_t sw, float* y, int64_t ldy, int64_t sy, int accumulate) {
    NS_TRY
    return gemm_h(g, "ns_gemm_batch_h", batch, trans_w, T, N, K, x, ldx, sx, w, ldw, sw, y, ldy, sy, accumulate);
    NS_CATCH
}

}  // extern "C"
