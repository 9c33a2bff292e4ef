#!/usr/bin/env python3
"""bench.py - the attention hot path on one MI355X, one JSON line on stdout.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload prefill8k|decode32k|...] [--no-cpu] [--no-extra]

A step is one pass of the hot path over one batch of synthetic input, inputs resident in HBM when the timed region
starts. The default workload is BASELINE.json's configs[1] - causal GQA flash-attention prefill, batch 1, 8192 rows, 40
query heads / 8 key heads, head 128, bfloat16 Q / K / V / output - and `value` is its TFLOP/s counted on the causal
flops 4 D Hq S (S + 1) / 2. The line also carries:
  roofline      the step's algorithmic flops (or bytes) over its device time - the median of 10 runs of steps between HIP
                event stamps on the library's own compute stream, every launch of a step included (a decode step's merge
                kernel too) - against MI355X's published peak; the dominant kernel alone from the committed kernel trace;
  cpu_baseline  the CPU oracle (a port of the reference's exact kernel, OpenMP) timed on this host on a bounded sample;
  others        the decode-side workloads of the same metric (GB/s of algorithmic KV bytes, % of 8 TB/s): the 32K GQA
                decode target, BASELINE configs 1, 3, 5 - unless --no-extra.
Decode workloads rotate over several distinct caches (> 512 MB in all) so the keys come from HBM, not from the 256 MB
Infinity Cache."""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS_BF16 = 2500.0   # MI355X dense bf16 / fp16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

# name -> (kind, T, Hq, Hkv, D, kv_len, kt, qt, description)
WORKLOADS = {
    "prefill8k": ("prefill", 8192, 40, 8, 128, 8192, 3, 2, "causal GQA flash-attention prefill, batch 1, seq 8192, 40 q heads / 8 kv heads, head_dim 128, bf16 (BASELINE configs[1])"),
    "decode4k": ("decode", 1, 32, 8, 128, 4096, 0, 1, "GQA decode, batch 1, 32 q heads / 8 kv heads, head_dim 128, KV 4096, f16 (BASELINE configs[0])"),
    "decode32k": ("decode", 1, 32, 8, 128, 32768, 0, 1, "GQA decode, batch 1, 32 q heads / 8 kv heads, head_dim 128, KV 32768, f16 (the north star's 32K target)"),
    "decode128k_q8": ("decode", 1, 64, 4, 128, 131072, 1, 1, "GQA decode, q8_0 KV cache, 64 q heads / 4 kv heads, head_dim 128, KV 131072 (BASELINE configs[2])"),
    "verify64k": ("decode", 4, 32, 4, 128, 65540, 0, 1, "MTP verify, 4 draft rows on a 65536-token f16 KV cache, 32 q heads / 4 kv heads, head_dim 128 (BASELINE configs[4])"),
    # MLA: Hq = heads, Hkv unused (one latent row a position), D = 512 latent + 64 rope
    "mla32k": ("mla", 1, 128, 1, 576, 32768, 0, 1, "DeepSeek-style absorbed MLA decode, 128 heads, 512 latent + 64 rope, f16 latent cache, KV 32768 (BASELINE configs[3])"),
    # the callers either side of the path: a prompt chunk through the latent MLA entry point (the reference's GEMM chain),
    # and the step in front of attention (q / k norm + rotary + KV store in one launch) at the prefill configuration
    "mla_prompt8k": ("mla", 256, 128, 1, 576, 8192 + 256, 0, 1, "absorbed MLA, a 256-row prompt chunk behind 8192 cells, 128 heads, f16 latent cache"),
    "pre_store8k": ("pre", 8192, 40, 8, 128, 8192, 3, 2, "q / k RMS norm + rotary + KV store, one launch, 8192 rows, 40 q / 8 kv heads of 128, bf16 rows and cache"),
}


GEN_SRC, GEN_LIB = os.path.join(ROOT, "bench_inputs.c"), os.path.join(ROOT, "bench_inputs.so")
_gen = None


def build_inputs(force=False):
    """Compile bench_inputs.c (gcc) into bench_inputs.so beside this script."""
    import subprocess
    if force or not os.path.exists(GEN_LIB) or os.path.getmtime(GEN_LIB) < os.path.getmtime(GEN_SRC):
        subprocess.run(["gcc", "-O3", "-ffp-contract=off", "-std=gnu11", "-shared", "-fPIC", GEN_SRC, "-o", GEN_LIB, "-lm"],
                       check=True, capture_output=True)
    return GEN_LIB


def _stream(seed, sigma, out):
    import ctypes as C
    global _gen
    if _gen is None:
        _gen = C.CDLL(build_inputs())
        _gen.bench_randn_f32.restype, _gen.bench_randn_f32.argtypes = None, [C.c_uint64, C.c_double, C.c_void_p, C.c_int64]
    _gen.bench_randn_f32(int(seed), float(sigma), out.ctypes.data, out.size)


GEN_ROWS = 1024


def randn(seed, shape, sigma=1.0):
    """Seeded N(0, sigma) float32: xorshift64* -> Box-Muller in float64 (bench_inputs.c), the generator the tests' inputs
    come from as well (there through the oracle's own statement of it). A vector is one stream in memory order; a matrix
    is a stream every GEN_ROWS rows, seeded seed + the block's first row (the streams are sequential: this is what lets
    the host's cores draw a few hundred million values in seconds)."""
    shape = tuple(int(d) for d in shape)
    out = np.empty(shape, np.float32)
    if len(shape) < 2 or shape[0] <= GEN_ROWS:
        _stream(seed, sigma, out.reshape(-1))
        return out
    from concurrent.futures import ThreadPoolExecutor
    rows = shape[0]
    flat = out.reshape(rows, -1)
    _stream(seed, sigma, flat[:min(GEN_ROWS, rows)].reshape(-1))          # (loads the generator before the threads start)
    with ThreadPoolExecutor(max_workers=min(16, os.cpu_count() or 1)) as ex:
        list(ex.map(lambda s0: _stream(seed + s0, sigma, flat[s0:min(rows, s0 + GEN_ROWS)].reshape(-1)), range(GEN_ROWS, rows, GEN_ROWS)))
    return out


def f2h(x):
    return np.ascontiguousarray(x, np.float32).astype(np.float16).view(np.uint16)


def f2bf(x):
    """float32 -> bfloat16 bits, round to nearest even."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def kv_bytes(kt, D):
    return {0: 2 * D, 1: D + D // 16, 2: D // 2 + D // 16, 3: 2 * D}[kt]


def algorithmic(kind, T, Hq, Hkv, D, kv, kt, qt):
    """(flops, bytes) of one step: the accounting of the reference's own probe (llm/qwen35/src/engine.rs:1540-1541,1591):
    flops 4 keys Hq D with keys = rows x visible keys; bytes = every visible K and V row once + q + out."""
    p0 = kv - T
    keys = T * p0 + T * (T + 1) // 2
    esz = 4 if qt == 0 else 2
    if kind == "mla":
        # scores over 576 features, the latent sum over 512; the cache once; q (576) and u (512) a head
        return 2 * keys * Hq * (576 + 512), kv * 576 * 2 + T * Hq * (576 + 512) * esz
    return 4 * keys * Hq * D, 2 * Hkv * kv * kv_bytes(kt, D) + 2 * T * Hq * D * esz


class Workload:
    """Synthetic inputs of one workload resident on the GPU: seeded N(0, 1) K / V rows packed by the library's own
    store kernel into `nbuf` distinct caches, query rows of the workload's type."""

    def __init__(self, ops, name, nbuf):
        from nextsycl_amd import DevBuf

        self.ops, self.name = ops, name
        self.kind, self.T, self.Hq, self.Hkv, self.D, self.kv, self.kt, self.qt, self.desc = WORKLOADS[name]
        g = ops.gpu
        T, Hq, Hkv, D, kv, kt, qt = self.T, self.Hq, self.Hkv, self.D, self.kv, self.kt, self.qt
        self.p0 = kv - T
        self.flops, self.bytes = algorithmic(self.kind, T, Hq, Hkv, D, kv, kt, qt)
        self.i = 0
        if self.kind == "pre":
            rb = kv_bytes(kt, D)
            self.bytes = T * (Hq + 2 * Hkv) * D * 4 + T * Hq * D * 2 + 2 * T * Hkv * rb       # float32 rows in; q rows, cache rows out
            self.flops = 0
            self.src = [DevBuf.of(g, randn(0xB0B + i, (T, h * D))) for i, h in enumerate((Hq, Hkv, Hkv))]
            self.w = [DevBuf.of(g, (1.0 + 0.1 * randn(0xD00D + i, (D,))).astype(np.float32)) for i in range(2)]
            self.out = DevBuf(g, T * Hq * D * 2)
            self.caches = [(DevBuf(g, Hkv * kv * rb), DevBuf(g, Hkv * kv * rb)) for _ in range(nbuf)]
            return
        if self.kind == "mla":
            self.caches = []
            host = f2h(randn(0xB0B, (kv, 576), 0.5))
            for b in range(nbuf):
                self.caches.append((DevBuf.of(g, host), None))
            self.q = DevBuf.of(g, f2h(randn(0xA11CE, (T, Hq, 576))))
            self.out = DevBuf(g, T * Hq * 512 * 2)
            self.scratch = DevBuf(g, 4 * ops.mla_latent_scratch(T, Hq, self.p0))
            return
        rb = kv_bytes(kt, D)
        self.caches = []
        chunk = 8192
        for b in range(nbuf):
            kc, vc = DevBuf(g, Hkv * kv * rb), DevBuf(g, Hkv * kv * rb)
            if b == 0:
                for s in range(0, kv, chunk):
                    n = min(chunk, kv - s)
                    k = DevBuf.of(g, randn(0xB0B + s, (n, Hkv * D)))
                    v = DevBuf.of(g, randn(0xC0FFEE + s, (n, Hkv * D)))
                    ops.kv_store(kt, k, Hkv * D, v, Hkv * D, n, Hkv, D, kv, s, kc, vc)
            else:
                # further caches: the same rows at other addresses (what the rotation needs is distinct memory)
                g.api.copy_dev(g.raw, kc.ptr, self.caches[0][0].ptr, kc.len)
                g.api.copy_dev(g.raw, vc.ptr, self.caches[0][1].ptr, vc.len)
            g.sync()
            self.caches.append((kc, vc))
        q = randn(0xA11CE, (T, Hq * D))
        qd = q if qt == 0 else (f2h(q) if qt == 1 else f2bf(q))
        self.q = DevBuf.of(g, qd)
        self.out = DevBuf(g, T * Hq * D * (4 if qt == 0 else 2))
        self.scratch = DevBuf(g, max(4, 4 * ops.decode_scratch(T, Hq, Hkv, D, self.p0))) if self.kind == "decode" else None

    def step(self):
        kc, vc = self.caches[self.i % len(self.caches)]
        self.i += 1
        o = self.ops
        if self.kind == "pre":
            q, k, v = self.src
            o.pre_store(1, self.qt, self.kt, False, q, self.Hq * self.D, self.D, self.out, self.Hq * self.D, k, self.Hkv * self.D, self.D, v,
                        self.Hkv * self.D, self.w[0], self.w[1], 1e-6, self.D // 2, 1e6, self.T, self.Hq, self.Hkv, self.D, self.kv, 0, kc, vc)
        elif self.kind == "mla":
            o.mla_decode_latent(1, self.q, kc, self.out, self.T, self.Hq, 64, self.p0, 192.0 ** -0.5, self.scratch)
        elif self.kind == "prefill":
            o.prompt(self.qt, self.kt, self.q, self.Hq * self.D, kc, vc, self.T, self.Hq, self.Hkv, self.D, self.kv, 0, self.out)
        else:
            o.decode(self.qt, self.kt, self.q, self.Hq * self.D, kc, vc, self.T, self.Hq, self.Hkv, self.D, self.kv, self.p0, self.out, self.scratch)


SETTLE_MS = 100.0
GROUPS = 10


def timed(w, steps, warmup):
    """(ms per step over exactly `steps` steps by the host's clock around two syncs; the step's device time in ns: the
    median over GROUPS runs of steps queued back to back between two HIP event stamps on the library's compute stream)."""
    g = w.ops.gpu
    # untimed: the W warmup steps, and then more of the same until the GPU has been under load for SETTLE_MS - an idle
    # MI355X takes tens of milliseconds of work to reach its steady clocks (the first MFMA-bound launches after a pause
    # run 15 - 30 % long), and the figure wanted is the sustained one
    for _ in range(warmup):
        w.step()
    g.sync()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < SETTLE_MS:
        for _ in range(8):
            w.step()
        g.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        w.step()
    g.sync()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    # the same steps on the device's clock: every launch of a step (main kernel, merge, a cache's widening) and the gaps
    # between dependent launches are inside; the median of GROUPS runs of `per` steps each
    per = max(10, steps // GROUPS)
    runs = []
    for _ in range(GROUPS):
        a = g.stamp()
        for _ in range(per):
            w.step()
        b = g.stamp()
        runs.append((a, b))
    dev = sorted(g.elapsed_ns(a, b) / per for a, b in runs)
    return ms, 0.5 * (dev[(GROUPS - 1) // 2] + dev[GROUPS // 2])


def kernel_events_us(w, n=30):
    """(dominant kernel, merge kernel) device time in us, each between two HIP events of its own on the compute stream
    (ns_attn_profile): the median of `n` steps. An event pair around one launch also spans the launch's start-up on the
    queue, so this reads a little longer than the kernel trace's duration of the same kernel. None for the workloads
    whose entry point sets no marks."""
    if w.kind == "pre" or (w.kind == "mla" and w.T > 256):         # (no marks; a longer prompt's passes would each overwrite them)
        return None
    ops = w.ops
    ops.profile(1)
    try:
        got = []
        for _ in range(n):
            w.step()
            got.append(ops.profile_last())
    except Exception:
        return None
    finally:
        ops.profile(0)
    med = lambda v: sorted(v)[len(v) // 2]
    return round(med([a for a, _ in got]) / 1e3, 2), round(med([b for _, b in got]) / 1e3, 2)


def graph_step_ms(w, n=50):
    """ms a step when `n` steps are captured into a HIP graph on the library's stream and replayed - how a serving loop
    queues a token's launches (no host call a kernel, the runtime hands the device the whole chain). Only for the
    workloads of two launches a step; None where the capture does not go through. The library records kernel launches
    only (no memset, no allocation), so the replay does what the calls did."""
    import ctypes as C
    if w.kind == "pre" or w.kind == "prefill" or (w.kind == "mla" and w.T > 16):
        return None
    g, k = w.ops.gpu, w.ops.k
    try:
        g.sync()
        h = C.c_void_p()
        if k.q35_graph_begin(g.raw, C.byref(h)) != 0:                 # ns_q35_graph_*: the library's stream capture
            return None
        try:
            for _ in range(n):
                w.step()
        finally:
            rc = k.q35_graph_end(g.raw, h)
        if rc != 0:
            k.q35_graph_free(h)
            return None
        try:
            for _ in range(3):
                k.q35_graph_launch(g.raw, h)
            g.sync()
            t0 = g.stamp()
            k.q35_graph_launch(g.raw, h)
            k.q35_graph_launch(g.raw, h)
            t1 = g.stamp()
            ns = g.elapsed_ns(t0, t1) / (2 * n)
        finally:
            g.sync()
            k.q35_graph_free(h)
        return ns / 1e6
    except Exception:
        return None


# What a profiler run says about each workload's dominant kernel: rocprofv3 cannot be driven from inside this script, so
# the figures are read from the committed summary of such a run of this script, profiles/<kernel>_<workload>.md - its
# lines "traffic_bytes_per_launch: N" (FETCH_SIZE + WRITE_SIZE per dispatch, each scaled by what the same counter reads
# for a plain copy kernel of known size) and "kernel_avg_us: T" (the kernel trace's average duration of that kernel) -
# and are null where no such summary exists.
def from_profile(kernel, workload, key):
    import re
    path = os.path.join(ROOT, "profiles", "%s_%s.md" % (kernel, workload))
    try:
        m = re.search(r"^%s:\s*([0-9.eE+]+)" % key, open(path).read(), re.M)
    except OSError:
        return None
    return float(m.group(1)) if m else None


KERNEL = {"pre": "pre_attn_kernel", "mla": "mla_decode_kernel", "prefill": "attn_prefill_kernel", "decode": "attn_decode_kernel"}


def roofline(w, step_ns):
    """The step against the roofline that bounds its dominant kernel. `achieved` / `frac`: algorithmic flops (or bytes) of
    the step over the step's device time, every launch of the step included (a decode step's merge kernel, a bfloat16
    cache's widening in front of the prompt kernel). `kernel_us` / `frac_kernel`: the dominant kernel alone between two
    HIP events of its own, measured in this run (`merge_us`: the merge kernel likewise); `kernel_us_trace`: the same
    kernel's average duration in the committed kernel trace of this script."""
    kernel = KERNEL[w.kind]
    hbm = w.kind in ("pre", "decode")
    ach = w.bytes / step_ns if hbm else w.flops / step_ns / 1e3
    peak = PEAK_HBM_GBS if hbm else PEAK_TFLOPS_BF16
    r = {"bound": "hbm" if hbm else "mfma", "achieved": round(ach, 2), "peak": peak, "unit": "GB/s" if hbm else "TFLOP/s", "frac": round(ach / peak, 4),
         "traffic": from_profile(kernel, w.name, "traffic_bytes_per_launch"), "kernel": kernel, "step_us": round(step_ns / 1e3, 2)}
    if w.kind == "mla":
        r["hbm_GB/s"] = round(w.bytes / step_ns, 1)
    kev = getattr(w, "kev", None)
    if kev:
        r["kernel_us"] = kev[0]
        r["frac_kernel"] = round((w.bytes / kev[0] / 1e3 if hbm else w.flops / kev[0] / 1e6) / peak, 4)
        if kev[1]:
            r["merge_us"] = kev[1]
    kus = from_profile(kernel, w.name, "kernel_avg_us")
    if kus:
        r["kernel_us_trace"] = kus
    return r


def cpu_baseline(name):
    """The CPU oracle (the C restatement of the reference's exact kernels, OpenMP over rows x heads) on a bounded sample of
    the workload, timed on this host's cores: a few seconds a workload, so that the default run stays within minutes."""
    from oracle import orc

    kind, T, Hq, Hkv, D, kv, kt, qt, _ = WORKLOADS[name]
    if kind == "pre":
        # the q and k rows' norm + rotary (the C restatement, one thread) on the first rows; the store is left out
        rows = min(T, 1024)
        w = np.ones(D, np.float32)
        xq, xk = randn(0xB0B, (rows, Hq * D)), randn(0xB0C, (rows, Hkv * D))
        t0 = time.perf_counter()
        orc.q35_norm_rope(xq, rows, Hq, D, w, 1e-6, D // 2, 1e6, 0)
        orc.q35_norm_rope(xk, rows, Hkv, D, w, 1e-6, D // 2, 1e6, 0)
        dt = time.perf_counter() - t0
        return {"value": round(rows * (Hq + Hkv) * D * 8 / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "norm + rotary of the first %d of %d q and k rows (float32 in and out), no store" % (rows, T), "seconds": round(dt, 2)}
    if kind == "mla":
        # the restated kernel order (16 streams a (row, head), exp) on the last rows and a quarter of the heads
        rows, heads = min(T, 2), max(1, Hq // 4)
        cache = f2h(randn(0xB0B, (kv, 576), 0.5))
        qa = orc.h2f(f2h(randn(0xA11CE, (rows, heads, 576))))
        p0 = kv - rows
        t0 = time.perf_counter()
        orc.mla_decode_u(qa, cache, rows, heads, p0, 192.0 ** -0.5)
        dt = time.perf_counter() - t0
        flops = sum(2 * heads * (p0 + r + 1) * 1088 for r in range(rows))
        return {"value": round(flops / dt / 1e12, 5), "unit": "TFLOP/s", "cores": orc.threads(), "kind": "port",
                "sample": "the last %d of %d rows, %d of %d heads, the whole %d-cell cache, reference-order float32 kernel" % (rows, T, heads, Hq, kv),
                "seconds": round(dt, 2)}
    k = randn(0xB0B, (kv, Hkv * D))
    v = randn(0xC0FFEE, (kv, Hkv * D))
    kc, vc = orc.kv_store(kt, k, v, Hkv, D, kv, 0)
    if kind == "prefill":
        rows = 1024          # the last 1024 query rows against the whole cache (~10-20 s on 16 cores)
        p0 = kv - rows
        q = orc.bf2f(f2bf(randn(0xA11CE, (rows, Hq * D))))
        sample = "last %d of %d query rows (positions %d..%d), all %d heads, full %d-key cache, reference-order float32 kernel" % (rows, T, p0, kv - 1, Hq, kv)
        flops = 4 * D * Hq * (rows * p0 + rows * (rows + 1) // 2)
        t0 = time.perf_counter()
        orc.attn_exact(q, kc, vc, kt, rows, Hq, Hkv, D, kv, p0, groups=max(1, Hq // 4))
        dt = time.perf_counter() - t0
        return {"value": round(flops / dt / 1e12, 5), "unit": "TFLOP/s", "cores": orc.threads(), "kind": "port", "sample": sample, "seconds": round(dt, 2)}
    q = randn(0xA11CE, (T, Hq * D))
    flops, nbytes = algorithmic(kind, T, Hq, Hkv, D, kv, kt, qt)
    reps, dt = 0, 0.0
    t0 = time.perf_counter()
    while reps < 3 and dt < 5.0:
        orc.attn_exact(q, kc, vc, kt, T, Hq, Hkv, D, kv, kv - T, groups=max(1, Hq // 4))
        reps += 1
        dt = time.perf_counter() - t0
    return {"value": round(nbytes * reps / dt / 1e9, 3), "unit": "GB/s", "cores": orc.threads(), "kind": "port",
            "sample": "the whole workload, %d passes, reference-order float32 kernel" % reps, "seconds": round(dt, 2)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="prefill8k", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the decode-side workloads of the metric")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MiB",
                    help="first run a plain copy kernel of this many MiB 5 times (the known-size kernel rocprofv3 traffic counters are scaled against)")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (the path would shard by key head, or by context with a merge of partials across GPUs)" % a.gpus,
              file=sys.stderr)
        sys.exit(2)

    from nextsycl_amd import Gpu, library_path
    from nextsycl_amd.attn import Ops

    if not os.path.exists(library_path()):
        from nextsycl_amd.build import build
        build()
    g = Gpu.open(0)
    ops = Ops(g)

    if a.copy_probe:
        from nextsycl_amd import DevBuf
        n = a.copy_probe << 20
        src, dst = DevBuf(g, n), DevBuf(g, n)
        src.fill(0x5A)
        for _ in range(5):
            ops.copy_probe(dst, src, n)
        g.sync()
        del src, dst

    def run(name, steps, warmup):
        kind = WORKLOADS[name][0]
        # decode: rotate distinct caches totalling > 512 MB so the keys are read from HBM
        nbuf = 1 if kind == "prefill" else 16 if kind == "mla" else 4 if kind == "pre" else max(4, int(np.ceil(600e6 / (2 * WORKLOADS[name][3] * WORKLOADS[name][5] * kv_bytes(WORKLOADS[name][6], WORKLOADS[name][4])))))
        nbuf = min(nbuf, 40)
        w = Workload(ops, name, nbuf)
        ms, step_ns = timed(w, steps, warmup)
        w.kev = kernel_events_us(w)
        w.graph_ms = graph_step_ms(w)
        return w, ms, step_ns

    w, ms, step_ns = run(a.workload, a.steps, a.warmup)
    if w.kind == "pre":
        metric, unit, value = "pre-attention step HBM GB/s (algorithmic bytes), 1 MI355X", "GB/s", w.bytes / (ms * 1e-3) / 1e9
    elif w.kind == "mla":
        metric, unit, value = "MLA decode attention TFLOP/s, 1 MI355X", "TFLOP/s", w.flops / (ms * 1e-3) / 1e12
    elif w.kind == "prefill":
        metric, unit, value = "prefill attention TFLOP/s (causal flops), 1 MI355X", "TFLOP/s", w.flops / (ms * 1e-3) / 1e12
    else:
        metric, unit, value = "decode attention HBM GB/s (algorithmic KV bytes), 1 MI355X", "GB/s", w.bytes / (ms * 1e-3) / 1e9
    line = {
        "metric": metric, "value": round(value, 3), "unit": unit, "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {0: "f32", 1: "f16", 2: "bf16"}[w.qt] if w.kt in (0, 3) else "q8_0/f16",
        "data": "synthetic (seeded xorshift64* + Box-Muller N(0,1))",
        "config": {"workload": w.desc, "name": a.workload, "rows": w.T, "q_heads": w.Hq, "kv_heads": w.Hkv, "head_dim": w.D, "kv_len": w.kv,
                   "kv_form": {0: "f16", 1: "q8_0", 2: "q4_0", 3: "bf16"}[w.kt], "flops_per_step": w.flops, "bytes_per_step": w.bytes,
                   "untimed_settle_ms": SETTLE_MS},
        "tokens_per_s": round(w.T / (ms * 1e-3), 1),
        "roofline": roofline(w, step_ns),
    }
    if w.graph_ms:
        line["graph_ms_per_step"] = round(w.graph_ms, 5)
    del w
    if not a.no_extra:
        others = {}
        for name in ("decode32k", "decode4k", "decode128k_q8", "verify64k", "mla32k", "prefill8k", "mla_prompt8k", "pre_store8k"):
            if name == a.workload:
                continue
            ww, m2, k2 = run(name, max(10, a.steps), a.warmup)
            r = roofline(ww, k2)
            others[name] = {"ms_per_step": round(m2, 5), "step_" + ("TFLOP/s" if ww.kind not in ("decode", "pre") else "GB/s"):
                            round((ww.flops / (m2 * 1e-3) / 1e12) if ww.kind not in ("decode", "pre") else (ww.bytes / (m2 * 1e-3) / 1e9), 2), "roofline": r}
            if ww.graph_ms:
                others[name]["graph_ms_per_step"] = round(ww.graph_ms, 5)
            del ww
            if not a.no_cpu:
                others[name]["cpu_baseline"] = cpu_baseline(name)
        line["others"] = others
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline(a.workload)
    print(json.dumps(line))
    g.close()


if __name__ == "__main__":
    main()
