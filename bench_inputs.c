/* bench_inputs.c - the seeded input generator of bench.py, in C because the stream is sequential (a few hundred million
 * draws a run): xorshift64* as the reference's own kernel checks draw their inputs (llm/deepseek2/src/tools.rs:14-23:
 * x ^= x >> 12; x ^= x << 25; x ^= x >> 27; the top 24 bits of x * 0x2545F4914F6CDD1D as a uniform), two uniforms ->
 * Box-Muller in float64 (u1 = (k1 + 1) / 2^24 in (0, 1], u2 = k2 / 2^24; the cosine branch for element 2 i, the sine branch
 * for 2 i + 1), scaled by sigma, rounded to float32. Built by __graft_entry__.build() (gcc) into bench_inputs.so; the tests
 * hold it to the oracle's generator, which states the same rule independently. */
#include <math.h>
#include <stdint.h>

static inline uint32_t next24(uint64_t* s) {
    uint64_t x = *s;
    x ^= x >> 12;
    x ^= x << 25;
    x ^= x >> 27;
    *s = x;
    return (uint32_t) ((x * 0x2545F4914F6CDD1DULL) >> 40);
}

void bench_randn_f32(uint64_t seed, double sigma, float* out, int64_t n) {
    uint64_t s = seed;
    const double two_pi = 6.283185307179586476925286766559, inv = 1.0 / 16777216.0;
    for (int64_t i = 0; i < n; i += 2) {
        const double u1 = ((double) next24(&s) + 1.0) * inv, u2 = (double) next24(&s) * inv;
        const double r = sqrt(-2.0 * log(u1)), a = two_pi * u2;
        out[i] = (float) (sigma * r * cos(a));
        if (i + 1 < n) out[i + 1] = (float) (sigma * r * sin(a));
    }
}
