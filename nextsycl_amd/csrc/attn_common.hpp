// attn_common.hpp: MFMA operand types and small device helpers shared by the attention kernels (gfx950, wave64).
//
// v_mfma_f32_16x16x32_{f16,bf16}: D[16x16] += A[16x32] B[32x16]. Per lane l (n = l % 16, g = l / 16):
//   A operand: row m = n, the 8 values k = 8 g .. 8 g + 7        B operand: column n, the same 8 k
//   D / C:     column n, rows m = 4 g .. 4 g + 3 (4 floats)
// v_mfma_f32_32x32x16_{f16,bf16}: D[32x32] += A[32x16] B[16x32]. Per lane l (n = l % 32, g = l / 32):
//   A operand: row m = n, k = 8 g .. 8 g + 7                     B operand: column n, the same 8 k
//   D / C:     column n, rows m = 8 (i / 4) + 4 g + i % 4 for register i = 0..15
// ds_read_b64_tr_b16 (the transposing LDS read): in each group of 16 lanes, lane s supplies the address of 4
// consecutive 16-bit values; lane i receives element i % 4 of the rows of lanes i / 4, 4 + i / 4, 8 + i / 4, 12 + i / 4.
// With lane s pointing at &M[k0 + s / 4][m0 + 4 (s % 4)] of a row-major M[k][m], lane i receives M[k0 .. k0 + 3][m0 + i]:
// the four k of one m - an MFMA operand's packing read out of the other-major matrix.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

typedef short s8v __attribute__((ext_vector_type(8)));
typedef short s4v __attribute__((ext_vector_type(4)));
typedef _Float16 h8v __attribute__((ext_vector_type(8)));
typedef __bf16 b8v __attribute__((ext_vector_type(8)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

template <bool BF>
__device__ __forceinline__ f4v mfma16(s8v a, s8v b, f4v c) {
    if constexpr (BF) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8v, a), __builtin_bit_cast(b8v, b), c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8v, a), __builtin_bit_cast(h8v, b), c, 0, 0, 0);
}
template <bool BF>
__device__ __forceinline__ f16v mfma32(s8v a, s8v b, f16v c) {
    if constexpr (BF) return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(b8v, a), __builtin_bit_cast(b8v, b), c, 0, 0, 0);
    else return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8v, a), __builtin_bit_cast(h8v, b), c, 0, 0, 0);
}

// float -> the kernel's 16-bit operand type, round to nearest even
template <bool BF>
__device__ __forceinline__ short to16(float f) {
    if constexpr (BF) {
        const __bf16 b = (__bf16) f;
        return __builtin_bit_cast(short, b);
    } else {
        const _Float16 h = (_Float16) f;
        return __builtin_bit_cast(short, h);
    }
}

// the transposing LDS read of 4 x 16 bits
__device__ __forceinline__ s4v lds_read_tr16(void* lds_addr) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s4v*) lds_addr);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
// the largest of three numbers as one instruction (for values that are never NaN: fmaxf would first quieten each input)
__device__ __forceinline__ float max3f(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// Reductions over the 4 lanes {n, n + 16, n + 32, n + 48} that hold one query row's scores. The partner's value comes
// by v_permlane16_swap / v_permlane32_swap (vector instructions: given two copies of v they return, in every lane, the
// values of the even and the odd 16-lane row of its pair / of the lower and the upper half of the wave), not through LDS
// as a general shuffle does: no LDS round trip to wait for in the softmax's dependency chain. Same operands, same sums.
__device__ __forceinline__ void pair16(float v, float& a, float& b) {
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    a = __builtin_bit_cast(float, (uint32_t) r[0]);
    b = __builtin_bit_cast(float, (uint32_t) r[1]);
}
__device__ __forceinline__ void pair32(float v, float& a, float& b) {
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    a = __builtin_bit_cast(float, (uint32_t) r[0]);
    b = __builtin_bit_cast(float, (uint32_t) r[1]);
}
__device__ __forceinline__ float rows_max(float v) {
    float a, b;
    pair16(v, a, b);
    pair32(fmaxf(a, b), a, b);
    return fmaxf(a, b);
}
__device__ __forceinline__ float rows_sum(float v) {
    float a, b;
    pair16(v, a, b);
    pair32(a + b, a, b);
    return a + b;
}

// Reductions over all 64 lanes without LDS: lane pairs inside a row of 16 through DPP (quad permutes, then the mirror
// of 8 and of 16 lanes, which pair the two halves as well as an exclusive-or would), rows through the permlane swaps.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t) __builtin_amdgcn_update_dpp(0, (int) v, CTRL, 0xF, 0xF, true);
}
template <typename F>
__device__ __forceinline__ uint32_t wave_reduce_u32(uint32_t v, F f) {
    v = f(v, dpp_u32<0xB1>(v));        // quad_perm [1, 0, 3, 2]
    v = f(v, dpp_u32<0x4E>(v));        // quad_perm [2, 3, 0, 1]
    v = f(v, dpp_u32<0x141>(v));       // row_half_mirror
    v = f(v, dpp_u32<0x140>(v));       // row_mirror
    auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    v = f((uint32_t) r[0], (uint32_t) r[1]);
    r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return f((uint32_t) r[0], (uint32_t) r[1]);
}
__device__ __forceinline__ float wave_max(float v) {
    return __builtin_bit_cast(float, wave_reduce_u32(__builtin_bit_cast(uint32_t, v), [](uint32_t a, uint32_t b) {
        return __builtin_bit_cast(uint32_t, fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b)));
    }));
}
__device__ __forceinline__ float wave_sum(float v) {
    return __builtin_bit_cast(float, wave_reduce_u32(__builtin_bit_cast(uint32_t, v), [](uint32_t a, uint32_t b) {
        return __builtin_bit_cast(uint32_t, __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b));
    }));
}
// the sum over each row of 16 lanes, in every lane of the row
__device__ __forceinline__ float row16_sum(float v) {
    auto f = [](float x) { return __builtin_bit_cast(uint32_t, x); };
    auto g = [](uint32_t x) { return __builtin_bit_cast(float, x); };
    v += g(dpp_u32<0xB1>(f(v)));
    v += g(dpp_u32<0x4E>(f(v)));
    v += g(dpp_u32<0x141>(f(v)));
    return v + g(dpp_u32<0x140>(f(v)));
}
__device__ __forceinline__ int wave_min(int v) {
    return (int) wave_reduce_u32((uint32_t) v, [](uint32_t a, uint32_t b) { return (uint32_t) min((int) a, (int) b); });
}

// element i of a row of query / output type QT (0 float32, 1 half, 2 bfloat16)
template <int QT>
__device__ __forceinline__ float load_q(const void* p, int64_t i) {
    if constexpr (QT == 0) return reinterpret_cast<const float*>(p)[i];
    else if constexpr (QT == 1) return (float) reinterpret_cast<const _Float16*>(p)[i];
    else return (float) reinterpret_cast<const __bf16*>(p)[i];
}
template <int QT>
__device__ __forceinline__ void store_o(void* p, int64_t i, float v) {
    if constexpr (QT == 0) reinterpret_cast<float*>(p)[i] = v;
    else if constexpr (QT == 1) reinterpret_cast<_Float16*>(p)[i] = (_Float16) v;
    else reinterpret_cast<__bf16*>(p)[i] = (__bf16) v;
}
