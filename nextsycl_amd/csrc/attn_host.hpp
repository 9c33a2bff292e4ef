// attn_host.hpp: the host-side entry points the attention translation units share (not part of the C ABI).
#pragma once
#include <algorithm>
#include <cstddef>
#include <cstdint>

#include "ns_internal.hpp"

// What a decode pass may differ in beyond its shapes: causal 0 = every row sees to the pass's last key (a draft block);
// kfirst >= 0 = every row starts at that key (a block with one first key for all its rows) instead of at its own
// window's; scratch_floats > 0 = what the scratch holds when it is not sized by ns_attn_decode_scratch (a buffer of the
// library's, or one a caller sized by another rule); marks = record the profiling events around the kernels
struct DecodeExtra {
    int causal = 1;
    int64_t kfirst = -1;
    int64_t scratch_floats = 0;
    bool marks = true;
};

// attn_decode.hip: a checked decode / verify pass of 1..16 rows
int ns_attn_decode_any(ns_gpu* g, const char* who, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T,
                       int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, const DecodeExtra& x, float scale, void* out,
                       float* scratch);
constexpr int64_t DECODE_ROWS = 16;   // passes up to this many rows take the decode kernel
// attn_decode.hip: block-sparse decode over a position-major half cache (rows with block lists of their own)
int ns_attn_decode_sel(ns_gpu* g, const char* who, const float* q, const uint16_t* kc, const uint16_t* vc, const int32_t* sel, int64_t K,
                       float* out, int64_t T, int64_t Hq, int64_t Hkv, int64_t pos0, float scale, float* scratch, size_t scratch_floats);
// attn_decode.hip: the merge of [rows][ns][D + 2] partials (also the prompt kernel's key splits')
int ns_attn_merge_partials(ns_gpu* g, int64_t D, const float* part, int64_t ns, int qt, int64_t rows, void* out);
// attn_prefill.hip: a checked prompt pass; causal 0 = every row sees to the pass's last key; kfirst as above
int ns_attn_prompt_any(ns_gpu* g, const char* who, int qt, int kt, int pm, const void* q, int64_t qs, const void* kc, const void* vc, int64_t T,
                       int64_t Hq, int64_t Hkv, int64_t D, int64_t cap, int64_t p0, int64_t win, int causal, int64_t kfirst, float scale,
                       void* out);

// Tuning knobs, 0 = the library's own choice: work-groups a decode pass aims for, key splits and waves of a prompt pass,
// work-groups an MLA pass aims for, heads a wave of the pre-attention kernel, and whether a prompt pass over a bfloat16,
// q8_0 or q4_0 cache keeps the rows' own form in the kernel (1) or widens them to half first whenever they fit (2). Each starts from its environment variable
// (NS_DEC_WGS, NS_PREFILL_SPLITS, NS_PREFILL_WAVES, NS_MLA_WGS, NS_PRE_HPW, NS_PREFILL_BF16, NS_SCRATCH_MIB), read once, and changes only
// through ns_attn_tune
enum { NS_TUNE_DEC_WGS = 0, NS_TUNE_PREFILL_SPLITS = 1, NS_TUNE_PREFILL_WAVES = 2, NS_TUNE_MLA_WGS = 3, NS_TUNE_PRE_HPW = 4, NS_TUNE_PREFILL_BF16 = 5,
       NS_TUNE_SCRATCH_MIB = 6, NS_TUNE_KNOBS = 7 };
int64_t ns_tune_get(int knob);
// floats of the library's own scratch a pass may plan with: all of it, or knob 6's MiB (NS_SCRATCH_MIB: tests of the paths
// a pass takes when its rows or partials outgrow the scratch)
inline size_t ns_own_floats(const ns_gpu* g) {
    const int64_t mib = ns_tune_get(NS_TUNE_SCRATCH_MIB);
    return mib > 0 ? std::min<size_t>(g->own_scratch_floats, (size_t) mib << 18) : g->own_scratch_floats;
}
