// kv_formats.hpp: device helpers for the cache row formats and 16-bit float conversions (shared by the store and the
// attention kernels).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

// float -> half bits, round to nearest even (v_cvt_f16_f32 under the default rounding mode)
__device__ __forceinline__ uint16_t f32_to_f16(float f) {
    const _Float16 h = (_Float16) f;
    return __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ float f16_to_f32(uint16_t b) { return (float) __builtin_bit_cast(_Float16, b); }
// float -> bfloat16 bits, round to nearest even; NaN stays NaN
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    return __builtin_bit_cast(uint16_t, (__bf16) f);        // gfx950 converts in hardware (v_cvt_pk_bf16_f32)
}
__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __builtin_bit_cast(float, (uint32_t) b << 16); }

__host__ __device__ constexpr int64_t kv_row_bytes(int kt, int64_t D) {
    return kt == 1 ? D + D / 32 * 2 : kt == 2 ? D / 2 + D / 32 * 2 : 2 * D;
}

// value i of a cache row of form kt as float32: (float) q x (float) half scale for the quantized forms
__device__ __forceinline__ float kv_value_f32(const uint8_t* row, int kt, int D, int i) {
    if (kt == 0) return f16_to_f32(*reinterpret_cast<const uint16_t*>(row + 2 * i));
    if (kt == 3) return bf16_to_f32(*reinterpret_cast<const uint16_t*>(row + 2 * i));
    const int b = i / 32, j = i % 32;
    if (kt == 1) return (float) (int8_t) row[i] * f16_to_f32(*reinterpret_cast<const uint16_t*>(row + D + 2 * b));
    const uint8_t w = row[b * 16 + (j & 15)];
    return (float) ((int) (j < 16 ? w & 15 : w >> 4) - 8) * f16_to_f32(*reinterpret_cast<const uint16_t*>(row + D / 2 + 2 * b));
}

// 8 int8 in two words -> 8 halfs x scale, as an MFMA operand / LDS piece. Each product is exact in float32, so one
// rounding to half (what the reference stages: half((float) q * (float) d)). Two values an instruction: a byte b of
// q + 128 under the exponent byte 0x64 is the half 1024 + b exactly, minus 1152 is q exactly, and the half product q x d
// rounds once.
__device__ __forceinline__ uint32_t dq8x2(uint32_t x, uint32_t sel, _Float16 d) {
    typedef _Float16 h2v __attribute__((ext_vector_type(2)));
    const h2v off = {(_Float16) -1152.0f, (_Float16) -1152.0f}, dd = {d, d};
    return __builtin_bit_cast(uint32_t, (__builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x, sel)) + off) * dd);
}
typedef short dq_s8v __attribute__((ext_vector_type(8)));   // (the attention kernels' s8v)
__device__ __forceinline__ dq_s8v dq8x8(uint32_t w0, uint32_t w1, _Float16 d) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const uint32_t x0 = w0 ^ 0x80808080u, x1 = w1 ^ 0x80808080u;
    const u4 r = {dq8x2(x0, 0x04010400u, d), dq8x2(x0, 0x04030402u, d), dq8x2(x1, 0x04010400u, d), dq8x2(x1, 0x04030402u, d)};
    return __builtin_bit_cast(dq_s8v, r);
}
// 8 nibbles (bits sh .. sh + 3 of each byte of two words) -> 8 halfs (nibble - 8) x scale: the same two-a-time form,
// a nibble under the exponent byte being 1024 + nibble and 1032 taken off
__device__ __forceinline__ uint32_t dq4x2(uint32_t x, uint32_t sel, _Float16 d) {
    typedef _Float16 h2v __attribute__((ext_vector_type(2)));
    const h2v off = {(_Float16) -1032.0f, (_Float16) -1032.0f}, dd = {d, d};
    return __builtin_bit_cast(uint32_t, (__builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x, sel)) + off) * dd);
}
__device__ __forceinline__ dq_s8v dq4x8(uint32_t w0, uint32_t w1, int sh, _Float16 d) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const uint32_t x0 = (w0 >> sh) & 0x0f0f0f0fu, x1 = (w1 >> sh) & 0x0f0f0f0fu;
    const u4 r = {dq4x2(x0, 0x04010400u, d), dq4x2(x0, 0x04030402u, d), dq4x2(x1, 0x04010400u, d), dq4x2(x1, 0x04030402u, d)};
    return __builtin_bit_cast(dq_s8v, r);
}
