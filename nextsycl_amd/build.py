"""Builds libnextsycl-llm.so (the HIP kernels + the C ABI) in-tree with hipcc for gfx950.

    python -m nextsycl_amd.build [--force]

hipcc cross-compiles without a GPU; the built library (nextsycl_amd/lib/, git-ignored) is what tests, smoke() and
bench.py load. Every translation unit gets -Xclang -target-feature -Xclang -packed-fp32-ops (packed FP32 math off) and
kv_store.hip additionally -ffp-contract=off (bit-exact quantizers)."""
import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INC = os.path.join(os.path.dirname(HERE), "include")
OUT = os.path.join(HERE, "lib")
LIB = os.path.join(OUT, "libnextsycl-llm.so")

COMMON = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
          "-packed-fp32-ops", "-I", INC, "-I", CSRC, "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option"]
# source -> extra flags
SOURCES = {
    "ns_hip.cpp": [],
    "kv_store.hip": ["-ffp-contract=off"],
    "kv_rows.hip": [],
    "pre_attn.hip": ["-ffp-contract=off"],
    "attn_decode.hip": [],
    "indexer.hip": [],
    "attn_prefill.hip": [],
    "attn_probs.hip": [],
    "attn_api.cpp": [],
    "mla.hip": [],
    "gemm_h.hip": [],
}


def _sources():
    return {s: f for s, f in SOURCES.items() if os.path.exists(os.path.join(CSRC, s))}


def _stale(obj, src):
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hpp", ".h"))] + [os.path.join(INC, f) for f in os.listdir(INC)]
    return any(os.path.getmtime(d) > t for d in [src] + deps)


def _compile(src, flags, force):
    path = os.path.join(CSRC, src)
    obj = os.path.join(OUT, os.path.splitext(src)[0] + ".o")
    if not force and not _stale(obj, path):
        return obj, ""
    cmd = ["hipcc"] + COMMON + flags + (["-x", "hip"] if src.endswith(".cpp") else []) + ["-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, r.stderr[-4000:]))
    return obj, r.stderr


def build(force=False, jobs=6):
    os.makedirs(OUT, exist_ok=True)
    srcs = _sources()
    with cf.ThreadPoolExecutor(max_workers=jobs) as ex:
        res = list(ex.map(lambda kv: _compile(kv[0], kv[1], force), srcs.items()))
    objs = [o for o, _ in res]
    if force or not os.path.exists(LIB) or any(os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs):
        cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode:
            raise RuntimeError("link failed:\n" + r.stderr[-4000:])
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
