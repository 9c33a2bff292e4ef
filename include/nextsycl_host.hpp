// nextsycl_host.hpp - the host side above the C ABI, in C++17 (header only; needs -ldl).
//
// What the reference keeps in Rust - the symbol table loaded with dlsym (crates/sys/src/lib.rs:62-64,138-237), GPUs and
// buffers that free themselves, bounds-checked copies and the per-pass bump arena (crates/core/src/lib.rs:13-44,133-236,
// 446-503), and an engine's table of attention entry points with the size-checked wrappers over it
// (llm/qwen35/src/ffi.rs:42-52,70-136, llm/deepseek2/src/ops.rs:391-445) - for hosts written in C++. Same names, same
// argument order, same ownership rules: the caller owns all device memory, kernels never allocate, an arena's views
// stay valid until it is rewound (the GPU's queue is in order), every failure is "<what>: <the library's reason>".
//
// Nothing here includes a HIP header or links the library: it is opened by name at run time, as the reference does.
#ifndef NEXTSYCL_HOST_HPP
#define NEXTSYCL_HOST_HPP

#include <dlfcn.h>

#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "ns.h"
#include "ns_attn.h"
#include "ns_mla.h"
#include "ns_pre.h"

namespace nextsycl {

// A failed call. no_room(): the one kind a caller may retry after freeing memory (crates/core/src/lib.rs:32-44)
class Error : public std::runtime_error {
public:
    explicit Error(const std::string& m) : std::runtime_error(m) {}
    static Error no_room(const std::string& m) { return Error("no room: " + m); }
    bool is_no_room() const {
        const std::string s = what();
        return s.rfind("no room: ", 0) == 0 || (s.find("device allocation of ") != std::string::npos && s.find(" bytes failed") != std::string::npos) ||
               s.find("hipErrorOutOfMemory") != std::string::npos || s.find("out of memory") != std::string::npos;
    }
};

// ---- the library: opened by name, every entry point looked up once (crates/sys/src/lib.rs:138-151,204-235) ----------

#define NS_HOST_DEVICE_SYMBOLS(X)                                                                                                        \
    X(ns_last_error) X(ns_version) X(ns_gpu_count) X(ns_gpu_name) X(ns_gpu_pci) X(ns_gpu_units) X(ns_gpu_open) X(ns_gpu_close)             \
    X(ns_gpu_queue) X(ns_gpu_memory) X(ns_alloc) X(ns_free) X(ns_alloc_host) X(ns_free_host) X(ns_copy_to) X(ns_copy_from) X(ns_copy_dev) \
    X(ns_copy_2d) X(ns_mark) X(ns_stream_copy) X(ns_await) X(ns_stamp) X(ns_elapsed) X(ns_fill) X(ns_sync) X(ns_copy_peer)

// the attention path: the reference's names (q35.h, mg.h, silo.h, mm3.h, ds2.h, glm.h) and this library's typed ones
#define NS_HOST_ATTN_SYMBOLS(X)                                                                                                          \
    X(ns_q35_kv_store) X(ns_q35_kv_store_q) X(ns_q35_attn_scratch) X(ns_q35_attn) X(ns_q35_attn_prompt_supported) X(ns_q35_attn_prompt)  \
    X(ns_q35_attn_prompt_kv) X(ns_q35_attn_decode_supported) X(ns_q35_attn_decode_scratch) X(ns_q35_attn_decode) X(ns_q35_attn_decode_kv) \
    X(ns_mg_kv_store) X(ns_mg_attn_scratch) X(ns_mg_attn) X(ns_mg_attn_prompt_supported) X(ns_mg_attn_prompt)                            \
    X(ns_mg_attn_decode_supported) X(ns_mg_attn_decode_scratch) X(ns_mg_attn_decode) X(ns_llm_minimaxm3_attend)                          \
    X(ns_rc_kv_store) X(ns_rc_attn_scratch) X(ns_rc_attn) X(ns_nh_kv_store) X(ns_nh_attn_scratch) X(ns_nh_attn)                          \
    X(ns_q35_graph_begin) X(ns_q35_graph_end) X(ns_q35_graph_launch) X(ns_q35_graph_free) \
    X(ns_rc_flash_prompt_supported) X(ns_rc_flash_prompt) X(ns_rc_flash_decode_supported) X(ns_rc_flash_decode_scratch) X(ns_rc_flash_decode) \
    X(ns_nhs_attn_prompt_supported) X(ns_nhs_attn_prompt) X(ns_nhs_attn_decode_supported) X(ns_nhs_attn_decode_scratch)                  \
    X(ns_nhs_attn_decode)                                                                                                                \
    X(ns_attn_kv_store) X(ns_attn_decode_scratch) X(ns_attn_decode_t) X(ns_attn_prompt_t) X(ns_attn_decode_static)                       \
    X(ns_ds2_rope) X(ns_ds2_kv_store) X(ns_ds2_mla_decode) X(ns_ds2_mla_decode_q6k) X(ns_mla_decode_latent_scratch) X(ns_mla_decode_latent)             \
    X(ns_mla_attend) X(ns_mla_attend_sel) X(ns_mla_attend_sel_q8) X(ns_to_q8row) X(ns_gather_q8_h)                                     \
    X(ns_idx_pool) X(ns_idx_score) X(ns_topk) X(ns_mla_cells) X(ns_softmax_masked) X(ns_gemm_f16) X(ns_gemm_batch_h) X(ns_to_f16) X(ns_gather_h)

class Api {
public:
#define NS_HOST_FIELD(name) decltype(&::name) name = nullptr;
    NS_HOST_DEVICE_SYMBOLS(NS_HOST_FIELD)
    NS_HOST_ATTN_SYMBOLS(NS_HOST_FIELD)
#undef NS_HOST_FIELD

    // NEXTSYCL_LIB, else `path`, else the name itself for the loader's own search (crates/sys/src/lib.rs:138-151)
    explicit Api(const std::string& path = "") {
        const char* env = std::getenv("NEXTSYCL_LIB");
        file_ = env && *env ? env : !path.empty() ? path : "libnextsycl-llm.so";
        handle_ = dlopen(file_.c_str(), RTLD_NOW | RTLD_GLOBAL);
        if (!handle_) throw Error("opening " + file_ + ": " + dlerror());
        // a missing symbol fails the load, but for ns_copy_2d (crates/sys/src/lib.rs:204-235)
#define NS_HOST_BIND(name) name = reinterpret_cast<decltype(name)>(find(#name, std::string(#name) != "ns_copy_2d"));
        NS_HOST_DEVICE_SYMBOLS(NS_HOST_BIND)
        NS_HOST_ATTN_SYMBOLS(NS_HOST_BIND)
#undef NS_HOST_BIND
    }
    Api(const Api&) = delete;
    Api& operator=(const Api&) = delete;
    ~Api() {
        if (handle_) dlclose(handle_);
    }

    // any further entry point by name (an engine's own table: llm/<arch>/src/ffi.rs)
    template <class Fn>
    Fn symbol(const char* name) const {
        return reinterpret_cast<Fn>(find(name, true));
    }
    bool has(const char* name) const { return dlsym(handle_, name) != nullptr; }
    std::string error() const {
        const char* e = ns_last_error();
        return e ? e : "";
    }
    const std::string& file() const { return file_; }
    int symbols() const { return bound_; }

private:
    void* find(const char* name, bool required) const {
        void* p = dlsym(handle_, name);
        if (!p && required) throw Error(file_ + " has no " + name);
        if (p) ++bound_;
        return p;
    }
    void* handle_ = nullptr;
    std::string file_;
    mutable int bound_ = 0;
};

inline void check(const Api& a, int rc, const std::string& what) {
    if (rc != 0) throw Error(what + ": " + a.error());
}

// ---- one GPU with its in-order queue (crates/core/src/lib.rs:133-215) ------------------------------------------------

class Gpu {
public:
    Gpu(std::shared_ptr<const Api> api, int index) : api_(std::move(api)), index_(index) {
        const int n = api_->ns_gpu_count();
        if (index < 0 || index >= n) throw Error("no GPU " + std::to_string(index) + " (" + std::to_string(n) + " found)");
        check(*api_, api_->ns_gpu_open(index, &raw_), "opening GPU " + std::to_string(index));
        char buf[256] = {0};
        if (api_->ns_gpu_name(index, buf, sizeof buf) == 0) name_ = buf;
    }
    static std::shared_ptr<Gpu> open(std::shared_ptr<const Api> api, int index = 0) { return std::make_shared<Gpu>(std::move(api), index); }
    Gpu(const Gpu&) = delete;
    Gpu& operator=(const Gpu&) = delete;
    ~Gpu() {
        if (raw_) {
            api_->ns_sync(raw_);
            api_->ns_gpu_close(raw_);
        }
    }
    ns_gpu* raw() const { return raw_; }
    const Api& api() const { return *api_; }
    const std::string& name() const { return name_; }
    int index() const { return index_; }
    void sync() const { check(*api_, api_->ns_sync(raw_), "waiting for the GPU"); }
    // (total bytes, free bytes or -1 where the driver does not tell)
    std::pair<uint64_t, int64_t> memory() const {
        uint64_t t = 0;
        int64_t f = -1;
        check(*api_, api_->ns_gpu_memory(raw_, &t, &f), "the GPU's memory");
        return {t, f};
    }
    int64_t stamp() const {
        int64_t t = 0;
        check(*api_, api_->ns_stamp(raw_, &t), "a stamp");
        return t;
    }
    double elapsed_ns(int64_t t0, int64_t t1) const {
        double ns = 0;
        check(*api_, api_->ns_elapsed(raw_, t0, t1, &ns), "the time between two stamps");
        return ns;
    }

private:
    std::shared_ptr<const Api> api_;
    int index_;
    ns_gpu* raw_ = nullptr;
    std::string name_;
};

// ---- device memory (crates/core/src/lib.rs:217-318,364-444). A view does not own its bytes -----------------------------

class DevBuf {
public:
    DevBuf() = default;
    DevBuf(std::shared_ptr<Gpu> gpu, size_t len) : gpu_(std::move(gpu)), len_(len), owned_(true) {
        void* p = nullptr;
        check(gpu_->api(), gpu_->api().ns_alloc(gpu_->raw(), len ? len : 1, &p), "allocating " + std::to_string(len) + " bytes on " + gpu_->name());
        ptr_ = static_cast<uint8_t*>(p);
    }
    DevBuf(DevBuf&& o) noexcept { *this = std::move(o); }
    DevBuf& operator=(DevBuf&& o) noexcept {
        if (this != &o) {
            release();
            gpu_ = std::move(o.gpu_);
            ptr_ = o.ptr_;
            len_ = o.len_;
            owned_ = o.owned_;
            o.ptr_ = nullptr;
            o.len_ = 0;
            o.owned_ = false;
        }
        return *this;
    }
    DevBuf(const DevBuf&) = delete;
    DevBuf& operator=(const DevBuf&) = delete;
    ~DevBuf() { release(); }

    static DevBuf f32(const std::shared_ptr<Gpu>& g, size_t n) { return DevBuf(g, 4 * n); }
    template <class T>
    static DevBuf from(const std::shared_ptr<Gpu>& g, const std::vector<T>& v) {
        DevBuf b(g, v.size() * sizeof(T));
        b.write(0, v.data(), v.size() * sizeof(T));
        return b;
    }

    void* ptr() const { return ptr_; }
    float* fp() const { return reinterpret_cast<float*>(ptr_); }
    size_t len() const { return len_; }
    size_t floats() const { return len_ / 4; }
    const std::shared_ptr<Gpu>& gpu() const { return gpu_; }

    void bounds(size_t at, size_t n) const {
        if (at > len_ || n > len_ - at) throw Error("bytes " + std::to_string(at) + ".." + std::to_string(at + n) + " of a " + std::to_string(len_) + "-byte buffer");
    }
    DevBuf view(size_t at, size_t n) const {
        bounds(at, n);
        DevBuf v;
        v.gpu_ = gpu_;
        v.ptr_ = ptr_ + at;
        v.len_ = n;
        v.owned_ = false;
        return v;
    }
    // host bytes into [at, at + n), waiting (the source may be a temporary)
    void write(size_t at, const void* src, size_t n) const {
        bounds(at, n);
        check(gpu_->api(), gpu_->api().ns_copy_to(gpu_->raw(), ptr_ + at, src, n), "copying to the GPU");
        gpu_->sync();
    }
    void read(size_t at, void* dst, size_t n) const {
        bounds(at, n);
        check(gpu_->api(), gpu_->api().ns_copy_from(gpu_->raw(), dst, ptr_ + at, n), "copying from the GPU");
        gpu_->sync();
    }
    template <class T>
    std::vector<T> to() const {
        std::vector<T> v(len_ / sizeof(T));
        read(0, v.data(), v.size() * sizeof(T));
        return v;
    }
    void fill(uint8_t v) const { check(gpu_->api(), gpu_->api().ns_fill(gpu_->raw(), ptr_, v, len_), "filling"); }
    void copy_within(size_t at, const DevBuf& src, size_t src_at, size_t n) const {
        bounds(at, n);
        src.bounds(src_at, n);
        check(gpu_->api(), gpu_->api().ns_copy_dev(gpu_->raw(), ptr_ + at, src.ptr_ + src_at, n), "copying on the GPU");
    }

private:
    void release() {
        if (owned_ && ptr_ && gpu_) gpu_->api().ns_free(gpu_->raw(), ptr_);
        ptr_ = nullptr;
    }
    std::shared_ptr<Gpu> gpu_;
    uint8_t* ptr_ = nullptr;
    size_t len_ = 0;
    bool owned_ = false;
};

// ---- a pass's temporaries out of one allocation (crates/core/src/lib.rs:446-503): views at multiples of 256 bytes, valid
// until the arena is rewound past them

class Arena {
public:
    Arena(const std::shared_ptr<Gpu>& g, size_t bytes) : buf_(g, bytes) {}
    size_t len() const { return buf_.len(); }
    DevBuf bytes(size_t n) {
        const size_t at = (off_ + 255) / 256 * 256;
        if (at > buf_.len() || n > buf_.len() - at) throw Error::no_room("an arena of " + std::to_string(buf_.len()) + " bytes holds " + std::to_string(off_) + ", asked for " + std::to_string(n));
        off_ = at + n;
        if (off_ > peak_) peak_ = off_;
        return buf_.view(at, n);
    }
    DevBuf f32(size_t n) { return bytes(4 * n); }
    void reset() { off_ = 0; }
    size_t mark() const { return off_; }
    void rewind(size_t mark) {
        if (mark < off_) off_ = mark;
    }
    size_t peak() const { return peak_; }

private:
    DevBuf buf_;
    size_t off_ = 0, peak_ = 0;
};

// ---- the checked attention calls (an engine's ops.rs). Sizes in elements as the kernels take them; every buffer is
// checked against what the kernel reads and writes before the call (llm/deepseek2/src/ops.rs:409-445) -------------------

enum RowType { F32 = 0, F16 = 1, BF16 = 2 };                  // q / out rows
enum KvForm { KV_F16 = 0, KV_Q8_0 = 1, KV_Q4_0 = 2, KV_BF16 = 3 };   // cache rows (llm/qwen35/src/engine.rs:35-60)

inline size_t row_type_bytes(int qt) { return qt == F32 ? 4 : 2; }
inline size_t kv_row_bytes(int kt, size_t D) {
    switch (kt) {
        case KV_F16:
        case KV_BF16: return 2 * D;
        case KV_Q8_0: return D + D / 32 * 2;
        case KV_Q4_0: return D / 2 + D / 32 * 2;
        default: throw Error("a cache form 0 (half), 1 (q8_0), 2 (q4_0) or 3 (bfloat16)");
    }
}

class Ops {
public:
    explicit Ops(std::shared_ptr<Gpu> g) : gpu_(std::move(g)) {}
    const std::shared_ptr<Gpu>& gpu() const { return gpu_; }

    // k, v float32 rows [T][Hkv D] (ks / vs floats apart) into the caches' rows p0 .. p0 + T - 1; ring: slot = position % cap
    void kv_store(int kt, bool ring, const DevBuf& k, size_t ks, const DevBuf& v, size_t vs, size_t T, size_t Hkv, size_t D, size_t cap, size_t p0,
                  const DevBuf& kc, const DevBuf& vc) const {
        if (T == 0) return;
        need(k, ((T - 1) * ks + Hkv * D) * 4, "kv_store k");
        need(v, ((T - 1) * vs + Hkv * D) * 4, "kv_store v");
        need(kc, Hkv * cap * kv_row_bytes(kt, D), "kv_store k cache");
        need(vc, Hkv * cap * kv_row_bytes(kt, D), "kv_store v cache");
        ok(api().ns_attn_kv_store(raw(), kt, ring, k.fp(), (int64_t) ks, v.fp(), (int64_t) vs, (int64_t) T, (int64_t) Hkv, (int64_t) D, (int64_t) cap,
                                  (int64_t) p0, kc.ptr(), vc.ptr()),
           "kv_store");
    }
    size_t decode_scratch(size_t T, size_t Hq, size_t Hkv, size_t D, size_t p0, size_t win = 0) const {
        return (size_t) api().ns_attn_decode_scratch((int64_t) T, (int64_t) Hq, (int64_t) Hkv, (int64_t) D, (int64_t) p0, (int64_t) win);
    }
    // a decode or verify pass (1..16 rows) over head-major caches: rows of type qt at positions p0.., out in the same type
    void decode(int qt, int kt, const DevBuf& q, size_t qs, const DevBuf& kc, const DevBuf& vc, size_t T, size_t Hq, size_t Hkv, size_t D, size_t cap,
                size_t p0, size_t win, float scale, const DevBuf& out, const DevBuf& scratch) const {
        if (T == 0) return;
        need(q, ((T - 1) * qs + Hq * D) * row_type_bytes(qt), "decode q");
        need(kc, Hkv * cap * kv_row_bytes(kt, D), "decode k cache");
        need(vc, Hkv * cap * kv_row_bytes(kt, D), "decode v cache");
        need(out, T * Hq * D * row_type_bytes(qt), "decode out");
        need(scratch, decode_scratch(T, Hq, Hkv, D, p0, win) * 4, "decode scratch");
        ok(api().ns_attn_decode_t(raw(), qt, kt, 0, q.ptr(), (int64_t) qs, kc.ptr(), vc.ptr(), (int64_t) T, (int64_t) Hq, (int64_t) Hkv, (int64_t) D,
                                  (int64_t) cap, (int64_t) p0, (int64_t) win, scale, out.ptr(), scratch.fp()),
           "decode");
    }
    // a prompt pass (more than 16 rows), causal
    void prompt(int qt, int kt, const DevBuf& q, size_t qs, const DevBuf& kc, const DevBuf& vc, size_t T, size_t Hq, size_t Hkv, size_t D, size_t cap,
                size_t p0, size_t win, float scale, const DevBuf& out) const {
        if (T == 0) return;
        need(q, ((T - 1) * qs + Hq * D) * row_type_bytes(qt), "prompt q");
        need(kc, Hkv * cap * kv_row_bytes(kt, D), "prompt k cache");
        need(vc, Hkv * cap * kv_row_bytes(kt, D), "prompt v cache");
        need(out, T * Hq * D * row_type_bytes(qt), "prompt out");
        ok(api().ns_attn_prompt_t(raw(), qt, kt, 0, q.ptr(), (int64_t) qs, kc.ptr(), vc.ptr(), (int64_t) T, (int64_t) Hq, (int64_t) Hkv, (int64_t) D,
                                  (int64_t) cap, (int64_t) p0, (int64_t) win, scale, out.ptr()),
           "prompt");
    }
    // the reference's own call sequence for a museglimmer layer (llm/museglimmer/src/engine.rs:856-873): the route is asked
    // per call, scratch comes from the pass arena
    void mg_attention(const DevBuf& q, const DevBuf& kc, const DevBuf& vc, size_t T, size_t Hq, size_t Hkv, size_t D, size_t cap, size_t p0, size_t win,
                      const DevBuf& out, Arena& arena) const {
        if (T == 0) return;
        need(q, T * Hq * D * 4, "attention q");
        need(out, T * Hq * D * 4, "attention out");
        need(kc, Hkv * cap * 2 * D, "attention k cache");
        need(vc, Hkv * cap * 2 * D, "attention v cache");
        const Api& a = api();
        if (a.ns_mg_attn_decode_supported((int64_t) T, (int64_t) Hq, (int64_t) Hkv, (int64_t) D)) {
            const DevBuf s = arena.f32((size_t) a.ns_mg_attn_decode_scratch((int64_t) T, (int64_t) Hq, (int64_t) Hkv, (int64_t) D, (int64_t) p0, (int64_t) win));
            ok(a.ns_mg_attn_decode(raw(), q.fp(), kc.ptr(), vc.ptr(), (int64_t) T, (int64_t) Hq, (int64_t) Hkv, (int64_t) D, (int64_t) cap, (int64_t) p0,
                                   (int64_t) win, out.fp(), s.fp()),
               "attn_decode");
        } else if (a.ns_mg_attn_prompt_supported((int64_t) T, (int64_t) Hq, (int64_t) Hkv, (int64_t) D)) {
            ok(a.ns_mg_attn_prompt(raw(), q.fp(), kc.ptr(), vc.ptr(), (int64_t) T, (int64_t) Hq, (int64_t) Hkv, (int64_t) D, (int64_t) cap, (int64_t) p0,
                                   (int64_t) win, out.fp()),
               "attn_prompt");
        } else {
            const DevBuf s = arena.f32((size_t) a.ns_mg_attn_scratch((int64_t) T, (int64_t) Hq, (int64_t) Hkv, (int64_t) D, (int64_t) p0, (int64_t) win, 1));
            ok(a.ns_mg_attn(raw(), q.fp(), kc.ptr(), vc.ptr(), (int64_t) T, (int64_t) Hq, (int64_t) Hkv, (int64_t) D, (int64_t) cap, (int64_t) p0, (int64_t) win,
                            1, out.fp(), s.fp()),
               "attn");
        }
    }

    // ---- MLA (llm/deepseek2/src/ops.rs:409-445)
    struct Rope {
        float base = 10000.0f, freq_scale = 1.0f, ext_factor = 0.0f, mscale = 1.0f, corr0 = 0.0f, corr1 = 0.0f;
    };
    void mla_kv_store(const DevBuf& kv, const DevBuf& w, float eps, const DevBuf& cache, size_t T, size_t L, size_t R, size_t pos0, const Rope& r) const {
        if (T == 0) return;
        need(kv, T * (L + R) * 4, "kv_store kv");
        need(w, L * 4, "kv_store w");
        need(cache, (pos0 + T) * (L + R) * 2, "kv_store cache");
        ok(api().ns_ds2_kv_store(raw(), kv.fp(), w.fp(), eps, static_cast<uint16_t*>(cache.ptr()), (int64_t) T, (int64_t) L, (int64_t) R, (int64_t) pos0, r.base,
                                 r.freq_scale, r.ext_factor, r.mscale, r.corr0, r.corr1),
           "kv_store");
    }
    void mla_decode(const DevBuf& q, const DevBuf& kb, const DevBuf& vb, const DevBuf& cache, const DevBuf& out, size_t T, size_t H, size_t pos0, float scale) const {
        if (T == 0) return;
        need(q, T * H * 192 * 4, "mla_decode q");
        need(kb, H * 512 * 128 * 2, "mla_decode k_b");
        need(vb, H * 128 * 512 * 2, "mla_decode v_b");
        need(cache, (pos0 + T) * 576 * 2, "mla_decode cache");
        need(out, T * H * 128 * 4, "mla_decode out");
        ok(api().ns_ds2_mla_decode(raw(), q.fp(), static_cast<const uint16_t*>(kb.ptr()), static_cast<const uint16_t*>(vb.ptr()),
                                   static_cast<const uint16_t*>(cache.ptr()), out.fp(), (int64_t) T, (int64_t) H, (int64_t) pos0, scale),
           "mla_decode");
    }
    size_t mla_latent_scratch(size_t T, size_t H, size_t pos0) const {
        return (size_t) api().ns_mla_decode_latent_scratch((int64_t) T, (int64_t) H, (int64_t) pos0);
    }
    // absorbed rows qa [T][H][512 + R] of type qt over the latent cache -> u [T][H][512] in the same type
    void mla_decode_latent(int qt, const DevBuf& qa, const DevBuf& cache, const DevBuf& u, size_t T, size_t H, size_t R, size_t pos0, float scale,
                           const DevBuf& scratch) const {
        if (T == 0) return;
        need(qa, T * H * (512 + R) * row_type_bytes(qt), "mla_decode_latent qa");
        need(cache, (pos0 + T) * (512 + R) * 2, "mla_decode_latent cache");
        need(u, T * H * 512 * row_type_bytes(qt), "mla_decode_latent u");
        need(scratch, mla_latent_scratch(T, H, pos0) * 4, "mla_decode_latent scratch");
        ok(api().ns_mla_decode_latent(raw(), qt, qa.ptr(), static_cast<const uint16_t*>(cache.ptr()), u.ptr(), (int64_t) T, (int64_t) H, (int64_t) R,
                                      (int64_t) pos0, scale, scratch.fp()),
           "mla_decode_latent");
    }

private:
    const Api& api() const { return gpu_->api(); }
    ns_gpu* raw() const { return gpu_->raw(); }
    void ok(int rc, const char* what) const { check(api(), rc, what); }
    static void need(const DevBuf& b, size_t bytes, const char* what) {
        if (b.len() < bytes) throw Error(std::string(what) + ": " + std::to_string(bytes) + " bytes needed, the buffer has " + std::to_string(b.len()));
    }
    std::shared_ptr<Gpu> gpu_;
};

}  // namespace nextsycl
#endif
