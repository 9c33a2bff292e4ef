// kv_pack.hpp: the quantized cache rows' packers as device functions, shared by the stores. 8 lanes hold a block of 32
// values (lane ln of the 8: values 4 ln .. 4 ln + 3); every result is bit-exact against ggml's quantize_row_q8_0_ref /
// quantize_row_q4_0_ref rules, so the including file must be compiled with -ffp-contract=off (a fused multiply-add
// inside x * id would round differently).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

// q8_0: d = amax / 127, q = round-half-away(x / d). Returns this lane's 4 int8 as one word; d is the block's scale.
__device__ __forceinline__ uint32_t q8_0_pack4(const float xs[4], float& d) {
    float amax = fmaxf(fmaxf(fabsf(xs[0]), fabsf(xs[1])), fmaxf(fabsf(xs[2]), fabsf(xs[3])));
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    amax = fmaxf(amax, __shfl_xor(amax, 2));
    amax = fmaxf(amax, __shfl_xor(amax, 4));
    d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) w |= (uint32_t) (uint8_t) (int8_t) roundf(xs[j] * id) << (8 * j);
    return w;
}

// q4_0: the block's signed extreme is the value of the largest magnitude, the FIRST of a tie (the lanes carry
// (magnitude, index) and keep the lower index on equal magnitudes); d = extreme / -8, q = min(15, (int) (x / d + 8.5)).
// Byte j pairs value j (low nibble) with value j + 16 (high): lanes 0..3 of the 8 return the block's bytes 4 ln .. 4 ln + 3
// (a lane's 4 low nibbles meet lane + 4's 4 high nibbles through a shuffle); lanes 4..7 return nothing of use.
__device__ __forceinline__ uint32_t q4_0_pack4(const float xs[4], int ln, float& d) {
    float am = 0.0f, m = 0.0f;
    int at = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (fabsf(xs[j]) > am) { am = fabsf(xs[j]); m = xs[j]; at = ln * 4 + j; }
    if (am == 0.0f) at = 32;   // no value yet: loses every tie
#pragma unroll
    for (int o = 1; o < 8; o <<= 1) {
        const float am2 = __shfl_xor(am, o), m2 = __shfl_xor(m, o);
        const int at2 = __shfl_xor(at, o);
        if (am2 > am || (am2 == am && at2 < at)) { am = am2; m = m2; at = at2; }
    }
    d = m / -8.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    uint32_t nib = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int qv = (int) (xs[j] * id + 8.5f);
        qv = qv > 15 ? 15 : qv;
        nib |= (uint32_t) qv << (8 * j);
    }
    const uint32_t hi = __shfl_xor(nib, 4);   // lanes 0..3 hold values 0..15 (low nibbles), 4..7 values 16..31
    return nib | (hi << 4);
}
