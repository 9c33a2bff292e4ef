// kv_store.hip: float32 k / v rows into the KV caches (half, bfloat16, q8_0, q4_0 rows), the caches' rows widened back
// to float32, and the 32-point Walsh-Hadamard rotation. Byte and integer work: every result here is bit-exact against
// ggml's quantize_row_q8_0_ref / quantize_row_q4_0_ref rules, so the file is compiled with -ffp-contract=off (a fused
// multiply-add inside x * id would round differently).
//
// Layout in HBM: head-major caches [Hkv][cap][row bytes]; a quantized row keeps its D/32 half scales BEHIND its values
// (q8_0: [D int8][D/32 half], q4_0: [D/2 bytes][D/32 half]) so a row's values are one aligned run for the attention
// kernels' 8- and 16-byte loads.
#include "ns_internal.hpp"
#include "ns_attn.h"
#include "kv_formats.hpp"
#include "kv_pack.hpp"

namespace {

// ---- half / bfloat16 stores: a thread four consecutive features of one (row t, head h): one 16-byte read, one 8-byte
// write, both coalesced across a wave
template <bool BF16>
__global__ void kv_store16_kernel(const float* __restrict__ k, int64_t ks, const float* __restrict__ v, int64_t vs, int64_t T, int64_t Hkv,
                                  int64_t D, int64_t cap, int64_t p0, int ring, uint16_t* __restrict__ kc, uint16_t* __restrict__ vc) {
    const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x, D4 = D / 4;
    if (i >= T * Hkv * D4) return;
    const int64_t d = (i % D4) * 4, h = (i / D4) % Hkv, t = i / (D4 * Hkv);
    const int64_t slot = ring ? (p0 + t) % cap : p0 + t, at = (h * cap + slot) * D + d;
    const float4 kf = *reinterpret_cast<const float4*>(k + t * ks + h * D + d);
    const float4 vf = *reinterpret_cast<const float4*>(v + t * vs + h * D + d);
    ushort4 ko, vo;
    if (BF16) {
        ko = make_ushort4(f32_to_bf16(kf.x), f32_to_bf16(kf.y), f32_to_bf16(kf.z), f32_to_bf16(kf.w));
        vo = make_ushort4(f32_to_bf16(vf.x), f32_to_bf16(vf.y), f32_to_bf16(vf.z), f32_to_bf16(vf.w));
    } else {
        ko = make_ushort4(f32_to_f16(kf.x), f32_to_f16(kf.y), f32_to_f16(kf.z), f32_to_f16(kf.w));
        vo = make_ushort4(f32_to_f16(vf.x), f32_to_f16(vf.y), f32_to_f16(vf.z), f32_to_f16(vf.w));
    }
    *reinterpret_cast<ushort4*>(kc + at) = ko;
    *reinterpret_cast<ushort4*>(vc + at) = vo;
}

// ---- q8_0 / q4_0 stores: 8 lanes a block of 32 values (a lane 4 consecutive floats); the packers are kv_pack.hpp's
template <int KT>
__global__ void kv_store_q_kernel(const float* __restrict__ k, int64_t ks, const float* __restrict__ v, int64_t vs, int64_t T, int64_t Hkv,
                                  int64_t D, int64_t cap, int64_t p0, uint8_t* __restrict__ kc, uint8_t* __restrict__ vc) {
    const int64_t gi = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;   // a multiple of 8 threads a block: no partial groups
    const int64_t nb = D / 32, total = 2 * T * Hkv * nb * 8;
    const bool live = gi < total;
    int64_t i = live ? gi : total - 1;
    const int ln = (int) (i % 8);
    i /= 8;
    const int64_t b = i % nb;
    i /= nb;
    const int64_t h = i % Hkv;
    i /= Hkv;
    const int64_t t = i % T;
    const bool isv = i / T == 1;
    const float* x = (isv ? v + t * vs : k + t * ks) + h * D + b * 32 + ln * 4;
    const int64_t rb = KT == 1 ? D + nb * 2 : D / 2 + nb * 2;
    uint8_t* row = (isv ? vc : kc) + (h * cap + p0 + t) * rb;
    const float4 xv = *reinterpret_cast<const float4*>(x);
    const float xs[4] = {xv.x, xv.y, xv.z, xv.w};
    float d;
    if (KT == 1) {
        const uint32_t w = q8_0_pack4(xs, d);
        if (live) {
            *reinterpret_cast<uint32_t*>(row + b * 32 + ln * 4) = w;
            if (ln == 0) *reinterpret_cast<uint16_t*>(row + D + 2 * b) = f32_to_f16(d);
        }
    } else {
        const uint32_t w = q4_0_pack4(xs, ln, d);
        if (live && ln < 4) {
            *reinterpret_cast<uint32_t*>(row + b * 16 + ln * 4) = w;
            if (ln == 0) *reinterpret_cast<uint16_t*>(row + D / 2 + 2 * b) = f32_to_f16(d);
        }
    }
}

__global__ void kv_dequant_kernel(int kt, const uint8_t* __restrict__ rows, int64_t n, int64_t D, int64_t stride, float* __restrict__ out) {
    const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n * D) return;
    out[i] = kv_value_f32(rows + (i / D) * stride, kt, (int) D, (int) (i % D));
}

__global__ void fwht32_kernel(float* __restrict__ x, int64_t rows, int64_t nb, int64_t stride) {
    const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * nb) return;
    float* p = x + (i / nb) * stride + (i % nb) * 32;
    float v[32];
#pragma unroll
    for (int j = 0; j < 32; ++j) v[j] = p[j];
#pragma unroll
    for (int o = 1; o < 32; o <<= 1)
#pragma unroll
        for (int j = 0; j < 32; ++j)
            if (!(j & o)) {
                const float a = v[j], c = v[j + o];
                v[j] = a + c;
                v[j + o] = a - c;
            }
#pragma unroll
    for (int j = 0; j < 32; ++j) p[j] = v[j] * 0.17677669529663687f;
}

// a plain copy, 16 bytes a thread: the known-size kernel that hardware traffic counters are calibrated against
__global__ void copy_probe_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, int64_t n16) {
    const int64_t i = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) dst[i] = src[i];
}

inline unsigned blocks_for(int64_t n, int per) { return (unsigned) ((n + per - 1) / per); }

}  // namespace

extern "C" {

int ns_attn_kv_store(ns_gpu* g, int kt, int ring, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D,
                     int64_t cap, int64_t p0, void* kc, void* vc) {
    NS_TRY
    if (T <= 0) return 0;
    if (kt < 0 || kt > 3) return ns_fail("ns_attn_kv_store: a cache form 0 (half), 1 (q8_0), 2 (q4_0) or 3 (bfloat16)");
    if (Hkv <= 0 || D <= 0 || D % 32 || ks % 4 || vs % 4) return ns_fail("ns_attn_kv_store: heads of a multiple of 32, row strides a multiple of 4");
    if (p0 < 0 || cap <= 0) return ns_fail("ns_attn_kv_store: a position and a capacity");
    if (!g || !k || !v || !kc || !vc) return ns_fail("ns_attn_kv_store: a null buffer");
    if (ring && (kt == 1 || kt == 2)) return ns_fail("ns_attn_kv_store: ring caches are half or bfloat16");
    if (ring ? T > cap : p0 + T > cap) return ns_fail("ns_attn_kv_store: past the cache's capacity");
    if (((uintptr_t) k | (uintptr_t) v) % 16 || ((uintptr_t) kc | (uintptr_t) vc) % 8) return ns_fail("ns_attn_kv_store: rows 16-byte aligned, caches 8-byte aligned");
    NS_HIP(hipSetDevice(g->dev));
    if (kt == 0 || kt == 3) {
        const int64_t n = T * Hkv * (D / 4);
        if (kt == 0)
            kv_store16_kernel<false><<<blocks_for(n, 256), 256, 0, g->q>>>(k, ks, v, vs, T, Hkv, D, cap, p0, ring, (uint16_t*) kc, (uint16_t*) vc);
        else
            kv_store16_kernel<true><<<blocks_for(n, 256), 256, 0, g->q>>>(k, ks, v, vs, T, Hkv, D, cap, p0, ring, (uint16_t*) kc, (uint16_t*) vc);
    } else {
        const int64_t n = 2 * T * Hkv * (D / 32) * 8;
        if (kt == 1) kv_store_q_kernel<1><<<blocks_for(n, 256), 256, 0, g->q>>>(k, ks, v, vs, T, Hkv, D, cap, p0, (uint8_t*) kc, (uint8_t*) vc);
        else kv_store_q_kernel<2><<<blocks_for(n, 256), 256, 0, g->q>>>(k, ks, v, vs, T, Hkv, D, cap, p0, (uint8_t*) kc, (uint8_t*) vc);
    }
    NS_LAUNCHED("kv_store");
    return 0;
    NS_CATCH
}

int ns_q35_kv_store(ns_gpu* g, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D, int64_t cap, int64_t p0,
                    void* kc, void* vc) {
    if (T <= 0) return 0;
    if (p0 + T > cap) return ns_fail("ns_q35_kv_store: past the cache's capacity");
    return ns_attn_kv_store(g, 0, 0, k, ks, v, vs, T, Hkv, D, cap, p0, kc, vc);
}

int ns_q35_kv_store_q(ns_gpu* g, int kt, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D, int64_t cap,
                      int64_t p0, void* kc, void* vc) {
    if (T <= 0) return 0;
    if (kt != 1 && kt != 2) return ns_fail("ns_q35_kv_store_q: form 1 (q8_0) or 2 (q4_0)");
    if (p0 + T > cap) return ns_fail("ns_q35_kv_store_q: past the cache's capacity");
    return ns_attn_kv_store(g, kt, 0, k, ks, v, vs, T, Hkv, D, cap, p0, kc, vc);
}

int ns_mg_kv_store(ns_gpu* g, const float* k, const float* v, int64_t T, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, void* kc, void* vc) {
    if (T <= 0) return 0;
    if (T > cap) return ns_fail("ns_mg_kv_store: more rows than the cache's slots");
    return ns_attn_kv_store(g, 0, 1, k, Hkv * D, v, Hkv * D, T, Hkv, D, cap, p0, kc, vc);
}

int ns_rc_kv_store(ns_gpu* g, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D, int64_t R, int64_t p0,
                   void* kc, void* vc) {
    if (T <= 0) return 0;
    if (T > R) return ns_fail("ns_rc_kv_store: more rows than the ring holds");
    return ns_attn_kv_store(g, 0, 1, k, ks, v, vs, T, Hkv, D, R, p0, kc, vc);
}

int ns_nh_kv_store(ns_gpu* g, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D, int64_t cap, int64_t p0,
                   void* kc, void* vc) {
    if (T <= 0) return 0;
    if (p0 + T > cap) return ns_fail("ns_nh_kv_store: past the cache's capacity");
    return ns_attn_kv_store(g, 0, 0, k, ks, v, vs, T, Hkv, D, cap, p0, kc, vc);
}

int ns_attn_kv_dequant(ns_gpu* g, int kt, const void* rows, int64_t n, int64_t D, int64_t stride, float* out) {
    NS_TRY
    if (n <= 0) return 0;
    if (kt < 0 || kt > 3 || D <= 0 || D % 32) return ns_fail("ns_attn_kv_dequant: a cache form 0..3, rows of a multiple of 32");
    if (stride < kv_row_bytes(kt, D) || ((uintptr_t) rows | (uintptr_t) stride) % 2) return ns_fail("ns_attn_kv_dequant: rows at least a row apart, 2-byte aligned");
    if (!g || !rows || !out) return ns_fail("ns_attn_kv_dequant: a null buffer");
    NS_HIP(hipSetDevice(g->dev));
    kv_dequant_kernel<<<blocks_for(n * D, 256), 256, 0, g->q>>>(kt, (const uint8_t*) rows, n, D, stride, out);
    NS_LAUNCHED("kv_dequant");
    return 0;
    NS_CATCH
}

int ns_attn_copy_probe(ns_gpu* g, void* dst, const void* src, size_t bytes) {
    NS_TRY
    if (bytes == 0) return 0;
    if (bytes % 16 || ((uintptr_t) dst | (uintptr_t) src) % 16) return ns_fail("ns_attn_copy_probe: a multiple of 16 bytes, 16-byte aligned");
    NS_HIP(hipSetDevice(g->dev));
    copy_probe_kernel<<<blocks_for((int64_t) (bytes / 16), 256), 256, 0, g->q>>>((const uint4*) src, (uint4*) dst, (int64_t) (bytes / 16));
    NS_LAUNCHED("copy_probe");
    return 0;
    NS_CATCH
}

int ns_q35_fwht32(ns_gpu* g, float* x, int64_t rows, int64_t n, int64_t stride) {
    NS_TRY
    if (rows <= 0) return 0;
    if (n <= 0 || n % 32) return ns_fail("ns_q35_fwht32: rows of a multiple of 32");
    if (stride < n) return ns_fail("ns_q35_fwht32: rows at least a row apart");
    if (!g || !x) return ns_fail("ns_q35_fwht32: a null buffer");
    NS_HIP(hipSetDevice(g->dev));
    const int64_t nb = n / 32;
    fwht32_kernel<<<blocks_for(rows * nb, 256), 256, 0, g->q>>>(x, rows, nb, stride);
    NS_LAUNCHED("fwht32");
    return 0;
    NS_CATCH
}

}  // extern "C"
