// host_harness.cpp - a C++ host over include/nextsycl_host.hpp that drives the attention path the way the reference's
// engines do (llm/museglimmer/src/engine.rs:856-873: kv_store -> *_supported -> *_scratch from the pass arena -> attention,
// no synchronisation until results are read) and checks every result against the CPU oracle, reporting max-abs, relative
// L2 and cosine as the reference's own `kernels` check does (llm/deepseek2/src/tools.rs:25-36). TEST PROGRAM: it links
// the oracle and is not part of the library.
//
//   host_harness --symbols     opens the library and binds every entry point; touches no GPU
//   host_harness               runs the checks on GPU 0; exit status 0 when all pass
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "nextsycl_host.hpp"

extern "C" {
void orc_randn_f32(uint64_t seed, double sigma, float* out, int64_t n);
void orc_f2h_n(const float* x, uint16_t* y, int64_t n);
void orc_h2f_n(const uint16_t* x, float* y, int64_t n);
int64_t orc_kv_row_bytes(int kt, int64_t D);
int orc_kv_store(int kt, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int ring,
                 uint8_t* kc, uint8_t* vc);
int orc_kv_store_q(int kt, const float* k, int64_t ks, const float* v, int64_t vs, int64_t T, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, uint8_t* kc,
                   uint8_t* vc);
int orc_attn_f64(const float* q, int64_t qs, const uint8_t* kc, const uint8_t* vc, int kt, int pm, int64_t T, int64_t Hq, int64_t Hkv, int64_t D,
                 int64_t cap, int64_t p0, int64_t win, int causal, double scale, double* out);
int orc_ds2_kv_store(const float* kv, const float* w, float eps, uint16_t* cache, int64_t T, int64_t L, int64_t R, int64_t pos0, float freq_base,
                     float freq_scale, float ext_factor, float mscale, float corr0, float corr1);
void orc_mla_f64(const float* qa, const uint16_t* cache, double* u, int64_t T, int64_t H, int64_t L, int64_t R, int64_t pos0, double scale);
void orc_compare(const float* a, const double* b, int64_t n, double* max_abs, double* rel_l2, double* cosine);
}

using namespace nextsycl;

namespace {

int failures = 0;

void report(const char* name, bool ok, const std::string& detail) {
    std::printf("%-34s %s  %s\n", name, ok ? "ok  " : "FAIL", detail.c_str());
    std::fflush(stdout);
    if (!ok) ++failures;
}

std::vector<float> randn(uint64_t seed, double sigma, size_t n) {
    std::vector<float> v(n);
    orc_randn_f32(seed, sigma, v.data(), (int64_t) n);
    return v;
}

// float32 results against the float64 closed form, within the bound for 16-bit operands
void close_to(const char* name, const std::vector<float>& got, const std::vector<double>& want, double max_abs_tol = 2e-3, double rel_tol = 1e-3) {
    double ma = 0, rl = 0, cs = 0;
    orc_compare(got.data(), want.data(), (int64_t) got.size(), &ma, &rl, &cs);
    char buf[160];
    std::snprintf(buf, sizeof buf, "max-abs %.3e  rel-L2 %.3e  cosine %.6f", ma, rl, cs);
    report(name, got.size() == want.size() && ma <= max_abs_tol && rl <= rel_tol, buf);
}

struct Shape {
    size_t Hq, Hkv, D, cap;
};

// the caches of `cap` positions from seeded float32 rows, stored by the library in chunks as an engine's prompt would
// be, and compared bit for bit with the oracle's packing
void fill_caches(const Ops& ops, int kt, const Shape& s, uint64_t seed, const DevBuf& kc, const DevBuf& vc, std::vector<uint8_t>& hk, std::vector<uint8_t>& hv,
                 const char* name) {
    const auto g = ops.gpu();
    const size_t rb = kv_row_bytes(kt, s.D), w = s.Hkv * s.D;
    const std::vector<float> k = randn(seed, 1.0, s.cap * w), v = randn(seed + 1, 1.0, s.cap * w);
    hk.assign(s.Hkv * s.cap * rb, 0);
    hv.assign(s.Hkv * s.cap * rb, 0);
    if (kt == KV_F16 || kt == KV_BF16) orc_kv_store(kt, k.data(), (int64_t) w, v.data(), (int64_t) w, (int64_t) s.cap, (int64_t) s.Hkv, (int64_t) s.D, (int64_t) s.cap, 0, 0, hk.data(), hv.data());
    else orc_kv_store_q(kt, k.data(), (int64_t) w, v.data(), (int64_t) w, (int64_t) s.cap, (int64_t) s.Hkv, (int64_t) s.D, (int64_t) s.cap, 0, hk.data(), hv.data());
    const DevBuf kd = DevBuf::from(g, k), vd = DevBuf::from(g, v);
    const size_t chunk = 1000;                                  // (not a multiple of anything the kernel tiles by)
    for (size_t p0 = 0; p0 < s.cap; p0 += chunk) {
        const size_t T = std::min(chunk, s.cap - p0);
        ops.kv_store(kt, false, kd.view(p0 * w * 4, T * w * 4), w, vd.view(p0 * w * 4, T * w * 4), w, T, s.Hkv, s.D, s.cap, p0, kc, vc);
    }
    const std::vector<uint8_t> gk = kc.to<uint8_t>(), gv = vc.to<uint8_t>();
    report(name, gk == hk && gv == hv, "cache rows bit for bit (" + std::to_string(hk.size() * 2) + " bytes)");
}

void run_checks() {
    auto api = std::make_shared<const Api>();
    auto gpu = Gpu::open(api, 0);
    const Ops ops(gpu);
    Arena arena(gpu, 64u << 20);
    std::printf("library %s (%s), GPU 0: %s\n", api->file().c_str(), api->ns_version(), gpu->name().c_str());

    // ---- a decode token, then a verify pass, over half caches (32 query / 8 key heads of 128, 4096 positions)
    {
        const Shape s{32, 8, 128, 4096};
        const size_t rb = kv_row_bytes(KV_F16, s.D);
        DevBuf kc(gpu, s.Hkv * s.cap * rb), vc(gpu, s.Hkv * s.cap * rb);
        std::vector<uint8_t> hk, hv;
        fill_caches(ops, KV_F16, s, 0xB0B, kc, vc, hk, hv, "kv_store half");
        const size_t T = 4, p0 = s.cap - T, w = s.Hq * s.D;
        const std::vector<float> q = randn(0xA11CE, 1.0, T * w);
        const DevBuf qd = DevBuf::from(gpu, q);
        // one row, through the engine's route
        DevBuf o1 = DevBuf::f32(gpu, w);
        arena.reset();
        ops.mg_attention(qd.view(3 * w * 4, w * 4), kc, vc, 1, s.Hq, s.Hkv, s.D, s.cap, s.cap - 1, 0, o1, arena);
        std::vector<double> want(w);
        orc_attn_f64(q.data() + 3 * w, (int64_t) w, hk.data(), hv.data(), KV_F16, 0, 1, (int64_t) s.Hq, (int64_t) s.Hkv, (int64_t) s.D, (int64_t) s.cap,
                     (int64_t) s.cap - 1, 0, 1, 1.0 / std::sqrt((double) s.D), want.data());
        close_to("decode 1 row at 4096 keys", o1.to<float>(), want);
        // four rows in one pass: each equal to its own one-row pass bit for bit (cli/nextsycl/src/main.rs:967-989)
        DevBuf o4 = DevBuf::f32(gpu, T * w);
        arena.reset();
        ops.mg_attention(qd, kc, vc, T, s.Hq, s.Hkv, s.D, s.cap, p0, 0, o4, arena);
        const std::vector<float> all = o4.to<float>();
        bool same = true;
        for (size_t t = 0; t < T; ++t) {
            arena.reset();
            ops.mg_attention(qd.view(t * w * 4, w * 4), kc, vc, 1, s.Hq, s.Hkv, s.D, s.cap, p0 + t, 0, o1, arena);
            const std::vector<float> one = o1.to<float>();
            same = same && std::memcmp(one.data(), all.data() + t * w, w * 4) == 0;
        }
        report("verify: rows = their own passes", same, "4 rows, bit for bit");
        std::vector<double> want4(T * w);
        orc_attn_f64(q.data(), (int64_t) w, hk.data(), hv.data(), KV_F16, 0, (int64_t) T, (int64_t) s.Hq, (int64_t) s.Hkv, (int64_t) s.D, (int64_t) s.cap, (int64_t) p0, 0,
                     1, 1.0 / std::sqrt((double) s.D), want4.data());
        close_to("verify 4 rows", all, want4);
        // a prompt chunk behind 3000 tokens: the route goes to the prompt kernel
        const size_t TP = 96, pp = 3000;
        const std::vector<float> qp = randn(0xA11CE + 7, 1.0, TP * w);
        DevBuf op = DevBuf::f32(gpu, TP * w);
        const DevBuf qpd = DevBuf::from(gpu, qp);
        arena.reset();
        ops.mg_attention(qpd, kc, vc, TP, s.Hq, s.Hkv, s.D, s.cap, pp, 0, op, arena);
        std::vector<double> wantp(TP * w);
        orc_attn_f64(qp.data(), (int64_t) w, hk.data(), hv.data(), KV_F16, 0, (int64_t) TP, (int64_t) s.Hq, (int64_t) s.Hkv, (int64_t) s.D, (int64_t) s.cap, (int64_t) pp,
                     0, 1, 1.0 / std::sqrt((double) s.D), wantp.data());
        close_to("prompt 96 rows behind 3000", op.to<float>(), wantp);
    }
    // ---- q8_0 caches, half rows (64 query / 4 key heads)
    {
        const Shape s{64, 4, 128, 8192};
        const size_t rb = kv_row_bytes(KV_Q8_0, s.D), w = s.Hq * s.D;
        DevBuf kc(gpu, s.Hkv * s.cap * rb), vc(gpu, s.Hkv * s.cap * rb);
        std::vector<uint8_t> hk, hv;
        fill_caches(ops, KV_Q8_0, s, 0xB0B + 2, kc, vc, hk, hv, "kv_store q8_0");
        const std::vector<float> q = randn(0xA11CE + 2, 1.0, w);
        std::vector<uint16_t> qh(w);
        orc_f2h_n(q.data(), qh.data(), (int64_t) w);
        std::vector<float> qr(w);
        orc_h2f_n(qh.data(), qr.data(), (int64_t) w);
        DevBuf out(gpu, w * 2);
        arena.reset();
        const DevBuf sc = arena.f32(ops.decode_scratch(1, s.Hq, s.Hkv, s.D, s.cap - 1));
        const DevBuf qd = DevBuf::from(gpu, qh);
        ops.decode(F16, KV_Q8_0, qd, w, kc, vc, 1, s.Hq, s.Hkv, s.D, s.cap, s.cap - 1, 0, 0.0f, out, sc);
        const std::vector<uint16_t> oh = out.to<uint16_t>();
        std::vector<float> of(w);
        orc_h2f_n(oh.data(), of.data(), (int64_t) w);
        std::vector<double> want(w);
        orc_attn_f64(qr.data(), (int64_t) w, hk.data(), hv.data(), KV_Q8_0, 0, 1, (int64_t) s.Hq, (int64_t) s.Hkv, (int64_t) s.D, (int64_t) s.cap, (int64_t) s.cap - 1, 0, 1,
                     1.0 / std::sqrt((double) s.D), want.data());
        close_to("decode q8_0, half rows", of, want);
    }
    // ---- MLA: the latent cache's rows, then the absorbed decode over them (16 heads, 2048 cells)
    {
        const size_t H = 16, L = 512, R = 64, n = 2048;
        const std::vector<float> kv = randn(0xB0B + 3, 0.5, n * (L + R));
        std::vector<float> wn = randn(0xD00D, 0.1, L);
        for (auto& x : wn) x += 1.0f;
        Ops::Rope r;
        r.base = 10000.0f;
        DevBuf cache(gpu, n * (L + R) * 2);
        const DevBuf kvd = DevBuf::from(gpu, kv), wd = DevBuf::from(gpu, wn);
        ops.mla_kv_store(kvd, wd, 1e-6f, cache, n, L, R, 0, r);
        std::vector<uint16_t> hc(n * (L + R));
        orc_ds2_kv_store(kv.data(), wn.data(), 1e-6f, hc.data(), (int64_t) n, (int64_t) L, (int64_t) R, 0, r.base, r.freq_scale, r.ext_factor, r.mscale, r.corr0, r.corr1);
        const std::vector<uint16_t> gc = cache.to<uint16_t>();
        std::vector<float> gf(gc.size()), hf(hc.size());
        orc_h2f_n(gc.data(), gf.data(), (int64_t) gc.size());
        orc_h2f_n(hc.data(), hf.data(), (int64_t) hc.size());
        size_t lat_diff = 0, rope_far = 0;
        for (size_t i = 0; i < n; ++i)
            for (size_t j = 0; j < L + R; ++j) {
                const size_t at = i * (L + R) + j;
                if (j < L) lat_diff += gc[at] != hc[at];
                // (sin / cos come from the device's own library: a last bit of the half)
                else rope_far += std::fabs(gf[at] - hf[at]) > std::ldexp(std::fmax(std::fabs(gf[at]), std::fabs(hf[at])), -10) + 1e-6f;
            }
        report("ds2_kv_store", lat_diff == 0 && rope_far == 0, "latent half bit for bit, rotated half within a last bit");
        const size_t T = 2, pos0 = n - T;
        const std::vector<float> qa = randn(0xA11CE + 3, 1.0, T * H * (L + R));
        DevBuf u = DevBuf::f32(gpu, T * H * L);
        arena.reset();
        const DevBuf sc = arena.f32(ops.mla_latent_scratch(T, H, pos0));
        const float scale = 1.0f / std::sqrt(192.0f);
        const DevBuf qad = DevBuf::from(gpu, qa);
        ops.mla_decode_latent(F32, qad, cache, u, T, H, R, pos0, scale, sc);
        // (the kernel rounds the absorbed rows to half: the closed form gets the same rows)
        std::vector<uint16_t> qh(qa.size());
        std::vector<float> qr(qa.size());
        orc_f2h_n(qa.data(), qh.data(), (int64_t) qa.size());
        orc_h2f_n(qh.data(), qr.data(), (int64_t) qa.size());
        std::vector<double> want(T * H * L);
        orc_mla_f64(qr.data(), gc.data(), want.data(), (int64_t) T, (int64_t) H, (int64_t) L, (int64_t) R, (int64_t) pos0, (double) scale);
        close_to("mla_decode_latent 2 rows", u.to<float>(), want);
    }
    // ---- failures arrive as Error with the reason, before or from the library
    {
        const Shape s{8, 2, 128, 256};
        const size_t rb = kv_row_bytes(KV_F16, s.D), w = s.Hq * s.D;
        DevBuf kc(gpu, s.Hkv * s.cap * rb), vc(gpu, s.Hkv * s.cap * rb), q = DevBuf::f32(gpu, 17 * w), out = DevBuf::f32(gpu, 17 * w);
        auto refused = [&](const char* name, const char* needle, const std::function<void()>& f, bool no_room = false) {
            try {
                f();
                report(name, false, "no error");
            } catch (const Error& e) {
                report(name, std::strstr(e.what(), needle) != nullptr && e.is_no_room() == no_room, e.what());
            }
        };
        refused("short scratch is caught here", "decode scratch",
                [&] { ops.decode(F32, KV_F16, q, w, kc, vc, 1, s.Hq, s.Hkv, s.D, s.cap, 100, 0, 0.0f, out, DevBuf(gpu, 16)); });
        refused("17 rows: the library says why", "1..16 rows", [&] {
            const DevBuf sc(gpu, 1u << 20);
            check(gpu->api(), gpu->api().ns_attn_decode_t(gpu->raw(), F32, KV_F16, 0, q.ptr(), (int64_t) w, kc.ptr(), vc.ptr(), 17, (int64_t) s.Hq, (int64_t) s.Hkv,
                                                          (int64_t) s.D, (int64_t) s.cap, 100, 0, 0.0f, out.ptr(), sc.fp()),
                  "decode");
        });
        refused("a full arena is 'no room'", "no room", [&] { Arena small(gpu, 4096); small.bytes(4000); small.bytes(4000); }, true);
    }
    gpu->sync();
}

}  // namespace

int main(int argc, char** argv) {
    try {
        if (argc > 1 && std::string(argv[1]) == "--symbols") {
            const Api api;
            std::printf("%s: %d entry points bound, version %s\n", api.file().c_str(), api.symbols(), api.ns_version());
            return 0;
        }
        run_checks();
    } catch (const std::exception& e) {
        std::printf("FAIL: %s\n", e.what());
        return 2;
    }
    std::printf(failures ? "%d check(s) failed\n" : "all checks passed\n", failures);
    return failures ? 1 : 0;
}
