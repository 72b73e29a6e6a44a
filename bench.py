#!/usr/bin/env python3
"""Benchmark of the ug HIP backend on one MI355X.

Headline (the JSON line): BASELINE config 2 -- sum(a*b + 0.5*a) over two f32 vectors of length
2^24, built as one lazy graph, scheduled and lowered like ug does, run on the HIP device.  A "step"
is one run of the compiled schedule (one kernel launch) with a and b resident in HBM.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--headline-only]

The other single-GPU configs (softmax sweep, batched matmul, llama pieces, llama decode) are
reported under "extras" of the same line; --headline-only (or --no-extras / --no-llama) leaves
them out, which is what the profiler runs use.  Only one GPU is ever used.
"""
import argparse
import contextlib
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0           # MI355X HBM3E, vendor figure
MFMA_BF16_PEAK_TF = 2500.0      # dense bf16
MFMA_F32_PEAK_TF = 157.3        # f32 matrix
N = 1 << 24
ALGO_BYTES = 2 * N * 4 + 4      # read a, read b, write one f32

# HBM bytes per step from `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE`, scaled by the counters' reading for the
# --copy-probe kernel.  A run of bench.py cannot read those counters itself: the figure is the one recorded in the
# profile named here, taken with the command that file gives, and the line says so.
TRAFFIC_BYTES = 134212407
TRAFFIC_SOURCE = "profiles/fused_reduce_2pow24_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE; not measured by this run)"


def hip_events(dev):
    import ug_amd
    lib = ug_amd.ughip_lib()
    raw = C.c_void_p(dev.raw_hip())
    evs = []
    for _ in range(2):
        e = C.c_void_p()
        assert lib.ughip_event_create(raw, C.byref(e)) == 0, lib.ughip_last_error()
        evs.append(e)
    return lib, evs


def timed(dev, fn, steps, warmup):
    """(wall seconds, HIP-event milliseconds) for `steps` calls of fn after `warmup` calls."""
    lib, (e0, e1) = hip_events(dev)
    for _ in range(warmup):
        fn()
    dev.synchronize()
    t0 = time.perf_counter()
    lib.ughip_event_record(e0)
    for _ in range(steps):
        fn()
    lib.ughip_event_record(e1)
    dev.synchronize()
    wall = time.perf_counter() - t0
    ms = C.c_float()
    assert lib.ughip_event_elapsed_ms(e0, e1, C.byref(ms)) == 0, lib.ughip_last_error()
    lib.ughip_event_destroy(e0)
    lib.ughip_event_destroy(e1)
    return wall, float(ms.value)


def timed_hot(dev, fn, steps, warmup, hot_s=0.25):
    """`timed` behind at least `hot_s` seconds of the same launches: the products below are each preceded by seconds of host
    work (operands, the float64 check), the chip falls back to its idle clocks meanwhile and takes a few hundred launches
    to come back up (measured: 4096^3 116 us per launch at first, 90 us from the 200th launch on)."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < hot_s:
        for _ in range(10):
            fn()
        dev.synchronize()
    return timed(dev, fn, steps, warmup)


# One wave reads the shader-clock counter and the constant 100 MHz counter, waits 20 us of the latter and reads both again:
# the ratio is the core clock the chip runs at when the probe executes, i.e. right behind whatever was queued in front of it.
CLOCK_PROBE_SRC = r"""
extern "C" __global__ void bench_clock_probe(long long* out) {
  const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  unsigned long long r1 = r0;
  for (int i = 0; i < (1 << 20) && r1 - r0 < 2000; ++i) { __builtin_amdgcn_s_sleep(8); r1 = __builtin_amdgcn_s_memrealtime(); }
  const unsigned long long c1 = __builtin_amdgcn_s_memtime();
  if (threadIdx.x == 0) { out[0] = (long long)(c1 - c0); out[1] = (long long)(r1 - r0); }
}
"""


class ClockProbe:
    def __init__(self, dev):
        import ug_amd
        self.lib, self.raw, self.dev = ug_amd.ughip_lib(), C.c_void_p(dev.raw_hip()), dev
        self.f = C.c_void_p()
        dts = (C.c_int * 1)(ug_amd.I64)
        assert self.lib.ughip_compile_source(self.raw, CLOCK_PROBE_SRC.encode(), b"bench_clock_probe", C.c_size_t(1), dts, C.c_uint(1), C.c_uint(64), C.c_uint(0), C.byref(self.f)) == 0, self.lib.ughip_last_error()
        self.out = dev.slice_from(np.zeros(2, np.int64))
        self.args = (C.c_void_p * 1)(C.c_void_p(self.out.raw()))

    def mhz(self):
        """Queues the probe behind what is already on the stream and waits for it."""
        assert self.lib.ughip_run(self.raw, self.f, self.args, C.c_size_t(1)) == 0, self.lib.ughip_last_error()
        c, r = self.out.to_vec()
        return round(float(c) / max(float(r), 1.0) * 100.0, 1)


def sustained_trace(dev, fn, seconds, block=50):
    """`fn` launched without a pause for `seconds`, HIP events on the library's stream every `block` launches and no
    synchronisation until the end: microseconds per launch of every block against the time since the first launch, averaged
    over buckets of 5 ms (the first 50 ms) and 50 ms.  Shows how the rate of one and the same step moves while the chip stays busy."""
    import ug_amd
    lib = ug_amd.ughip_lib()
    raw = C.c_void_p(dev.raw_hip())
    n_blocks = max(4, int(seconds / (block * 20e-6)))
    evs = []
    for _ in range(n_blocks + 1):
        e = C.c_void_p()
        assert lib.ughip_event_create(raw, C.byref(e)) == 0, lib.ughip_last_error()
        evs.append(e)
    dev.synchronize()
    lib.ughip_event_record(evs[0])
    for i in range(n_blocks):
        for _ in range(block):
            fn()
        lib.ughip_event_record(evs[i + 1])
    dev.synchronize()
    ms = C.c_float()
    t, rows = 0.0, []
    for i in range(n_blocks):
        assert lib.ughip_event_elapsed_ms(evs[i], evs[i + 1], C.byref(ms)) == 0, lib.ughip_last_error()
        rows.append((t, float(ms.value) * 1e3 / block))
        t += float(ms.value)
    for e in evs:
        lib.ughip_event_destroy(e)
    buckets = {}
    for t0, us in rows:
        buckets.setdefault(5 * int(t0 // 5) if t0 < 50 else 50 * int(t0 // 50), []).append(us)
    return [{"from_ms": k, "us_per_step": round(sum(v) / len(v), 3), "GB/s": round(ALGO_BYTES / (sum(v) / len(v)) / 1e3, 1), "blocks": len(v)} for k, v in sorted(buckets.items())]


def fused_reduce(dev, a, b):
    from ug_amd import LazyBuffer as LB, Schedule
    from ug_amd.graphs import fused_reduce_graph
    la, lb = LB.copy(a, (a.size,), dev), LB.copy(b, (b.size,), dev)
    r = fused_reduce_graph(la, lb, dev)
    cs = Schedule.create_one(r).compile()
    return r, cs, (la, lb)


def fused_reduce_parts(dev, a, b, truth, steps, warmup):
    """The two kernels of the config-2 step timed one at a time: the same SSA the schedule hands to Device::compile,
    compiled once more and launched through ughip_run_part on resident operands.  Returns microseconds per launch of the
    first (partial sums: all the traffic) and the second (fold of one partial per workgroup) kernel."""
    import ug_amd
    from ug_amd import LazyBuffer as LB, Schedule
    from ug_amd.graphs import fused_reduce_graph
    n = a.size
    la, lb = LB.copy(a, (n,), dev), LB.copy(b, (n,), dev)
    sched = Schedule.create_one(fused_reduce_graph(la, lb, dev))
    func = dev.compile(sched.item_ssa(0), "bench_fused_reduce")
    sa, sb, dst = dev.slice_from(a), dev.slice_from(b), dev.allocate_uninit(ug_amd.F32, 1)
    dev.run(func, [sa, sb, dst])          # argument order = ascending ArgId: a, b, dst (schedule.rs:457-465)
    got = float(dst.to_vec()[0])
    if not abs(got - truth) <= 1e-5 * abs(truth) + 1e-2:
        raise RuntimeError(f"fused_reduce_parts: wrong result {got} vs {truth}")
    lib = ug_amd.ughip_lib()
    raw_dev, raw_f = C.c_void_p(dev.raw_hip()), C.c_void_p(func._raw())
    args = (C.c_void_p * 3)(sa.raw(), sb.raw(), dst.raw())
    out = []
    for part in (1, 2):
        def launch():
            rc = lib.ughip_run_part(raw_dev, raw_f, args, C.c_size_t(3), part)
            if rc:
                raise RuntimeError(lib.ughip_last_error().decode())
        _, ms = timed(dev, launch, steps, warmup)
        out.append(ms * 1e3 / steps)
    return out


def cpu_baseline(a, b, truth, budget_s=12.0):
    """The CPU oracle (restatement of ug's CPU backend: same emitted C, same gcc flags, one thread)
    on the same workload, timed on this box's host cores."""
    from oracle.load import cpu_device
    cpu = cpu_device()
    r, cs, keep = fused_reduce(cpu, a, b)
    cs.run()
    val = float(r.data_vec()[0])
    assert abs(val - truth) <= 1e-3 * abs(truth) + 1.0, (val, truth)
    passes, t0 = 0, time.perf_counter()
    while True:
        cs.run()
        passes += 1
        el = time.perf_counter() - t0
        if el > budget_s or passes >= 100000:
            break
    return {"value": round(ALGO_BYTES * passes / el / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{passes} passes of the full 2^24-element workload in {el:.1f} s (oracle/: C emitted as ug-core/src/cpu_code_gen.rs does, "
                      "gcc -O3 -march=native -ffast-math, single thread like the reference)",
            "host_cpus": os.cpu_count()}


def cpu_extras(budget_s=3.0):
    """The CPU oracle (restatement of ug's CPU backend) on configs 1, 3, 4 and 5, timed on this box's host
    cores next to the GPU numbers: each a bounded sample of the same workload."""
    from oracle.load import cpu_device, cpu_llama_ops
    import ug_amd
    from ug_amd import LazyBuffer as LB, Schedule, rng
    cpu = cpu_device()
    cpu_ops = cpu_llama_ops()
    out = {}

    def sample(run):
        run()
        n, t0 = 0, time.perf_counter()
        while True:
            run()
            n += 1
            el = time.perf_counter() - t0
            if el > budget_s:
                return n, el

    rows, cols = 32, 1024
    sm = ug_amd.llama.softmax(LB.copy(rng.normal(1, rows * cols, 3.0), (rows, cols), cpu))
    cs = Schedule.create_one(sm).compile()
    n, el = sample(cs.run)
    out["cpu_softmax_lazy_32x1024"] = {"us_per_softmax": round(el / n * 1e6, 1), "GB/s": round(8.0 * rows * cols * n / el / 1e9, 4), "cores": 1, "kind": "port",
                                       "sample": f"{n} runs of the two kernels the reference's lowering emits (max and sum recomputed per element) in {el:.1f} s"}
    b, m = 8, 1024
    threads = min(16, os.cpu_count() or 1)   # a one-GPU box's share of host cores
    os.environ.setdefault("RAYON_NUM_THREADS", str(threads))   # the oracle's matmul reads it, like the reference (utils.rs:3-20)
    a, w = rng.uniform_pm1(4, b * m * m), rng.uniform_pm1(5, b * m * m)
    mm = LB.copy(a, (b, m, m), cpu).matmul(LB.copy(w, (b, m, m), cpu))
    cs = Schedule.create_one(mm).compile()
    n, el = sample(cs.run)
    out["cpu_bmm_f32_8x1024^3"] = {"TFLOP/s": round(2.0 * b * m * m * m * n / el / 1e12, 4), "ms": round(el / n * 1e3, 1), "cores": int(os.environ["RAYON_NUM_THREADS"]), "kind": "port",
                                   "sample": f"{n} runs in {el:.1f} s; the reference multiplies with the gemm crate, the oracle with its own blocked loops"}
    # config 4, the llama layer pieces at T = 512 (f32): the custom ops and the two products at full size; the lazy-graph
    # kernels (RMSNorm, softmax) recompute their reductions for every element like the reference's (2048^2 and 512^2
    # iterations per row), so a few rows are timed and scaled to the 512 / 16384 rows of the config
    t, hidden, heads, hd = 512, 2048, 32, 64
    ll = ug_amd.llama

    def c4(name, lb, nbytes, scale=1.0, note=""):
        cs = Schedule.create_one(lb).compile()
        n, el = sample(cs.run)
        sec = el / n * scale
        out[name] = {"ms": round(sec * 1e3, 3), "GB/s": round(nbytes / sec / 1e9, 3), "algorithmic_bytes": nbytes, "cores": 1, "kind": "port",
                     "sample": f"{n} runs in {el:.1f} s" + (f"; {note}" if note else "")}

    rows = 8
    c4("cpu_c4_rms_norm_512x2048", ll.rms_norm(LB.copy(rng.normal(6, rows * hidden), (1, rows, hidden), cpu), LB.copy(rng.normal(106, hidden, 0.02), (hidden,), cpu), 1e-5),
       2 * 4 * t * hidden + 4 * hidden, t / rows, f"{rows} of the 512 rows timed, scaled by {t // rows}")
    cfg = ug_amd.LlamaConfig()
    cos, sin = ll.rope_tables(cpu, cfg)
    cos.realize()
    sin.realize()
    q = LB.copy(rng.normal(7, heads * t * hd), (1, heads, t, hd), cpu)
    pos = LB.copy(np.zeros(1, np.int32), (1,), cpu)
    c4("cpu_c4_rope_q_1x32x512x64", cpu_ops.rope(q, cos, sin, pos), 2 * 4 * heads * t * hd + 2 * 4 * t * (hd // 2))
    sc = LB.copy(rng.normal(8, heads * t * t), (1, heads, t, t), cpu)
    c4("cpu_c4_causal_mask_1x32x512x512", cpu_ops.causal_mask(sc), 2 * 4 * heads * t * t)
    c4("cpu_c4_softmax_custom_1x32x512x512", cpu_ops.custom_softmax(sc), 2 * 4 * heads * t * t)
    rows = 4
    c4("cpu_c4_softmax_lazy_1x32x512x512", ll.softmax(LB.copy(rng.normal(8, rows * t), (1, 1, rows, t), cpu)), 2 * 4 * heads * t * t, heads * t / rows,
       f"{rows} of the 16384 rows timed, scaled by {heads * t // rows}")
    kk = LB.copy(rng.normal(208, heads * t * hd), (1, heads, t, hd), cpu)
    v = LB.copy(rng.normal(308, heads * t * hd), (1, heads, t, hd), cpu)
    for name, mm, flop in (("cpu_c4_qk_t_b32_512x512x64", q.matmul_t(kk), 2.0 * heads * t * t * hd), ("cpu_c4_att_v_b32_512x64x512", sc.matmul(v), 2.0 * heads * t * hd * t)):
        cs = Schedule.create_one(mm).compile()
        n, el = sample(cs.run)
        out[name] = {"ms": round(el / n * 1e3, 3), "TFLOP/s": round(flop * n / el / 1e12, 4), "cores": int(os.environ["RAYON_NUM_THREADS"]), "kind": "port", "sample": f"{n} runs in {el:.1f} s"}
    # config 5 at full width, two of the 22 layers: a decode step is the same two layers 11 times over
    # plus the head, so the per-layer and the head time are fitted from a 1-layer and a 2-layer run
    prompt = rng.token_ids(10, 8, 32000)
    n_steps = 6
    per_tok = {}
    for layers in (1, 2):
        cfg = ug_amd.LlamaConfig(num_hidden_layers=layers)
        model = ug_amd.LlamaModel(cpu, cpu_ops, cfg, custom_softmax=True, seed=9, std=0.02)
        model.generate(prompt, 1)     # compiles (gcc) every kernel once
        _, st = model.generate(prompt, n_steps)
        per_tok[layers] = st["decode_ms"] / n_steps
        del model
    layer_ms = per_tok[2] - per_tok[1]
    full_ms = per_tok[1] + 21 * layer_ms
    out["cpu_llama_decode_f32"] = {"tok/s": round(1e3 / full_ms, 3), "decode_ms_per_token": round(full_ms, 1), "ms_per_layer": round(layer_ms, 2),
                                   "ms_1_layer_model": round(per_tok[1], 2), "ms_2_layer_model": round(per_tok[2], 2), "cores": int(os.environ["RAYON_NUM_THREADS"]),
                                   "kind": "port", "sample": f"{n_steps} decode steps each of a 1-layer and a 2-layer model of config 5's width after an 8-token prompt; "
                                   "22 layers = the 1-layer step + 21 x the difference (the fused kernels run on one thread as in the reference, the matmuls on all)"}
    return out


def extras(dev, steps, warmup, only=None):
    """Other single-GPU configs of BASELINE.json: GB/s or TFLOP/s with the roofline fraction.  A group that fails (a check
    that does not hold, a launch error) is reported under `<group>_error` and does not take the other groups down."""
    out = {}
    groups = (("softmax", lambda: softmax_sweep(dev, steps, warmup)), ("bmm", lambda: bmm(dev, steps, warmup)),
              ("llama_pieces", lambda: llama_pieces(dev, steps, warmup)), ("hbm_large", lambda: hbm_large(dev, steps, warmup)),
              ("floors", lambda: launch_and_barrier_floors(dev)), ("safetensors", lambda: safetensors_load(dev)), ("cpu", cpu_extras))
    for name, run in groups:
        if only not in (None, name):
            continue
        try:
            out.update(run())
        except Exception as e:  # noqa: BLE001
            out[f"{name}_error"] = f"{type(e).__name__}: {e}"
    return out


FLOOR_CHAIN_SRC = r"""
extern "C" __global__ void bench_chain_step(const float* x, float* y) {
  const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
  y[i] = x[i] + 1.0f;
}
"""

# `iters` barriers inside one launch.  Arrivals go to 16 counters (workgroup % 16), every workgroup polls all 16;
# between barriers every workgroup hands a value to its neighbour through memory (stored and loaded at agent scope),
# so a barrier that lets someone through early shows up in stale[0].  A poll gives up after 2^22 rounds (gave_up[0]).
FLOOR_BARRIER_SRC = r"""
#define G 16
#define PAD 64
#define ITERS %d
__device__ __forceinline__ bool grid_barrier(unsigned* counters, unsigned target, unsigned* gave_up) {
  __syncthreads();
  if (threadIdx.x == 0) {
    __builtin_amdgcn_s_waitcnt(0);
    __hip_atomic_fetch_add(&counters[(blockIdx.x %% G) * PAD], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  bool ok = true;
  if (threadIdx.x < G) {
    unsigned spins = 0;
    while (__hip_atomic_load(&counters[threadIdx.x * PAD], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
      __builtin_amdgcn_s_sleep(1);
      if (++spins > (1u << 22) || __hip_atomic_load(gave_up, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) { ok = false; break; }
    }
    if (!ok) __hip_atomic_store(gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  return ok;
}
extern "C" __global__ void __launch_bounds__(256) bench_grid_barrier(unsigned* counters, float* data, unsigned* gave_up, unsigned* stale) {
  const unsigned n = gridDim.x;
  const unsigned hits = threadIdx.x < G ? (n - threadIdx.x + G - 1) / G : 0;  // workgroups that arrive at this thread's counter
  for (unsigned it = 0; it < ITERS; ++it) {
    if (threadIdx.x == 0) __hip_atomic_store(&data[blockIdx.x * 16], (float)(it + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (!grid_barrier(counters, hits * (it + 1), gave_up)) return;
    if (threadIdx.x == 0 && __hip_atomic_load(&data[((blockIdx.x + 1) %% n) * 16], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (float)(it + 1)) atomicAdd(stale, 1u);
  }
}
"""


# Nothing but bf16 MFMAs, one wave per SIMD on every CU, eight independent accumulators of 32 x 32: what the matrix pipes sustain
# for tens of milliseconds with operands in U(-1, 1) (random sign, mantissa and two exponent bits per element) and with zeros.
FLOOR_MFMA_SRC = r"""
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ unsigned two_bf16(unsigned& s) {
  s = s * 1664525u + 1013904223u;
  const unsigned lo = ((s >> 3) & 0x807f) | (0x3f00 - ((s >> 20) & 3) * 0x80), hi = ((s >> 13) & 0x807f) | (0x3f00 - ((s >> 26) & 3) * 0x80);
  return lo | (hi << 16);
}
extern "C" __global__ void __launch_bounds__(256) bench_mfma_only(float* out, const int* cfg) {
  const int iters = cfg[0], zeros = cfg[1];
  unsigned seed = blockIdx.x * 256 + threadIdx.x + 1;
  u32x4 a[8], b[8];
  for (int j = 0; j < 8; ++j) {
    a[j] = zeros ? u32x4{0, 0, 0, 0} : u32x4{two_bf16(seed), two_bf16(seed), two_bf16(seed), two_bf16(seed)};
    b[j] = zeros ? u32x4{0, 0, 0, 0} : u32x4{two_bf16(seed), two_bf16(seed), two_bf16(seed), two_bf16(seed)};
  }
  floatx16 acc[8];
  for (int q = 0; q < 8; ++q) for (int r = 0; r < 16; ++r) acc[q][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int q = 0; q < 8; ++q)
        acc[q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[(j + q) & 7]), __builtin_bit_cast(bf16x8, b[(j + 3 * q) & 7]), acc[q], 0, 0, 0);
  }
  float s = 0.f;
  for (int q = 0; q < 8; ++q) for (int r = 0; r < 16; ++r) s += acc[q][r];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}
"""


def launch_and_barrier_floors(dev):
    """What one dependent step costs on this box, the two ways a decode step can be cut into steps: (a) a chain of
    launches on one stream, each reading what the one before wrote; (b) a grid-wide barrier with a value handed over
    through memory inside one resident kernel, at 64 / 256 / 512 workgroups.  Both kernels are built from source
    through ughip_compile_source and run through ughip_run."""
    import ug_amd
    lib, raw = ug_amd.ughip_lib(), C.c_void_p(dev.raw_hip())
    out = {}

    def compile_src(src, entry, dtypes, grid, block):
        f = C.c_void_p()
        dts = (C.c_int * len(dtypes))(*dtypes)
        assert lib.ughip_compile_source(raw, src.encode(), entry.encode(), C.c_size_t(len(dtypes)), dts, C.c_uint(grid), C.c_uint(block), C.c_uint(0), C.byref(f)) == 0, lib.ughip_last_error()
        return f

    def run(f, slices):
        arr = (C.c_void_p * len(slices))(*[C.c_void_p(s_.raw()) for s_ in slices])
        assert lib.ughip_run(raw, f, arr, C.c_size_t(len(slices))) == 0, lib.ughip_last_error()

    # One thread issues a launch every ~3 us: the chain of tiny steps measures that rate (the GPU side of a small dependent
    # kernel, 1.2-2 us, is in the kernel traces under profiles/).
    for name, grid in (("launch_chain_8_workgroups", 8),):
        n = grid * 256
        a, b = dev.slice_from(np.zeros(n, np.float32)), dev.slice_from(np.zeros(n, np.float32))
        f = compile_src(FLOOR_CHAIN_SRC, "bench_chain_step", [ug_amd.F32, ug_amd.F32], grid, 256)
        ab = (C.c_void_p * 2)(C.c_void_p(a.raw()), C.c_void_p(b.raw()))
        ba = (C.c_void_p * 2)(C.c_void_p(b.raw()), C.c_void_p(a.raw()))
        go, two = lib.ughip_run, C.c_size_t(2)

        def burst():      # 100 launches with as little interpreter work between them as ctypes allows
            for _ in range(50):
                go(raw, f, ab, two)
                go(raw, f, ba, two)
        reps = 20
        wall, ms = timed(dev, burst, reps, 2)
        got = a.to_vec()
        if not np.all(got == 100.0 * (reps + 2)):
            raise RuntimeError(f"{name}: the chain lost a step ({got[:4]})")
        out[name] = {"us_per_dependent_launch": round(ms * 1e3 / (100 * reps), 2), "host_us_per_launch": round(wall * 1e6 / (100 * reps), 2),
                     "bytes_per_launch": 8 * n, "verified": True}
        lib.ughip_func_release(f)
    # The matrix pipes alone: 64 MFMAs of 32 x 32 x 16 per iteration and wave, 4 waves on each of 256 CUs
    mf_iters = 20000
    f = compile_src(FLOOR_MFMA_SRC, "bench_mfma_only", [ug_amd.F32, ug_amd.I32], 256, 256)
    sink = dev.slice_from(np.zeros(256 * 256, np.float32))
    for label, zeros in (("random", 0), ("zero", 1)):
        cfg = dev.slice_from(np.array([mf_iters, zeros], np.int32))
        run(f, [sink, cfg])
        _, ms = timed(dev, lambda: run(f, [sink, cfg]), 2, 0)
        got = sink.to_vec()
        if not np.all(np.isfinite(got)) or (zeros and np.any(got != 0.0)) or (not zeros and not np.any(got != 0.0)):
            raise RuntimeError(f"mfma only, {label} operands: unexpected sums")
        tf = 64.0 * 32768 * 4 * 256 * mf_iters * 2 / (ms * 1e-3) / 1e12
        out[f"mfma_bf16_only_{label}_operands"] = {"TFLOP/s": round(tf, 1), "frac_mfma_bf16": round(tf / MFMA_BF16_PEAK_TF, 4), "ms_per_launch": round(ms / 2, 1), "verified": True}
    lib.ughip_func_release(f)
    iters = 2000
    for wgs in (64, 256, 512):
        counters = dev.slice_from(np.zeros(16 * 64, np.int32))
        data = dev.slice_from(np.zeros(wgs * 16, np.float32))
        gave_up, stale = dev.slice_from(np.zeros(1, np.int32)), dev.slice_from(np.zeros(1, np.int32))
        f = compile_src(FLOOR_BARRIER_SRC % iters, "bench_grid_barrier", [ug_amd.I32, ug_amd.F32, ug_amd.I32, ug_amd.I32], wgs, 256)
        _, ms = timed(dev, lambda: run(f, [counters, data, gave_up, stale]), 1, 0)
        g, st = int(gave_up.to_vec()[0]), int(stale.to_vec()[0])
        if g or st or not np.all(data.to_vec()[::16] == float(iters)):
            raise RuntimeError(f"grid barrier at {wgs} workgroups: gave up {g}, stale reads {st}")
        out[f"grid_barrier_{wgs}_workgroups"] = {"us_per_barrier_and_handoff": round(ms * 1e3 / iters, 2), "barriers": iters, "counters": 16, "verified": True}
        lib.ughip_func_release(f)
    return out


def safetensors_load(dev, n=1 << 27):
    """A 256 MiB bf16 tensor in a safetensors file (page cache warm) loaded as f32: upload + widen
    on the device against widen on the host + upload (the order of ug-core/src/safetensors.rs:141-271),
    and the widening kernel alone (6 bytes per element)."""
    import tempfile
    from ug_amd import st_writer as st_files
    import ug_amd
    from ug_amd import rng
    out = {}
    bits = np.tile(rng.to_bf16_bits(rng.normal(11, 1 << 20)), n >> 20)
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "w.safetensors")
        st_files.write_safetensors(path, [("w", "BF16", (n,), bits)])
        st = ug_amd.Safetensors(path)
        for key, env in (("device_cast", None), ("host_cast", "1")):
            if env:
                os.environ["UG_SAFETENSORS_HOST_CAST"] = env
            try:
                st.load("w", dev, ug_amd.F32).data_vec()[:1]      # first touch: page in, warm the pool
                dev.synchronize()
                t0 = time.perf_counter()
                lb = st.load("w", dev, ug_amd.F32)
                dev.synchronize()
                dt = time.perf_counter() - t0
            finally:
                os.environ.pop("UG_SAFETENSORS_HOST_CAST", None)
            out[f"safetensors_bf16_to_f32_{key}"] = {"file_GB/s": round(2.0 * n / dt / 1e9, 2), "ms": round(dt * 1e3, 1), "on_device": st.last_cast_on_device}
            del lb
    src = dev.slice_from(bits)
    dst = dev.allocate_uninit(ug_amd.F32, n)
    _, ms = timed(dev, lambda: dev.convert(dst, src), 20, 3)
    gbs = 6.0 * n * 20 / (ms * 1e-3) / 1e9
    out["convert_bf16_to_f32_2pow27"] = {"GB/s": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4), "us": round(ms * 1e3 / 20, 1), "algorithmic_bytes": 6 * n}
    return out


def softmax_sweep(dev, steps, warmup):
    import ug_amd
    from ug_amd import LazyBuffer as LB, Schedule, rng
    out = {}
    # config 1 and the reference's own sweep (ug-cuda/examples/benchmark.rs:110): 8 B per element
    for rows, cols in [(32, 1024)] + [(4096, c) for c in (128, 256, 512, 768, 1024, 1536, 2048, 3072, 4096)]:
        x = rng.normal(1, rows * cols, 3.0)
        src = LB.copy(x, (rows, cols), dev)
        sm = ug_amd.llama.softmax(src)
        cs = Schedule.create_one(sm).compile()
        _, ms = timed(dev, cs.run, steps, warmup)
        gbs = 8.0 * rows * cols * steps / (ms * 1e-3) / 1e9
        out[f"softmax_lazy_{rows}x{cols}"] = {"GB/s": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4), "us_per_softmax": round(ms * 1e3 / steps, 2),
                                             "launches": 2}
        # the scheduler (unchanged from the reference) splits the softmax at the exp buffer: the pair moves 16 B per element for the 8
        # algorithmic ones, so half the roofline is its ceiling, whatever the two kernels do
        out[f"softmax_lazy_{rows}x{cols}"]["moved_bytes_per_element"] = 16
        if rows * cols * 8 < (1 << 22):   # under 4 MiB the bytes take well under a microsecond at 8 TB/s: what is measured is launches
            out[f"softmax_lazy_{rows}x{cols}"]["bound"] = "2 launch floors (the scheduler splits the softmax at the exp buffer); HBM time of these bytes is %.3f us" % (rows * cols * 8 / HBM_PEAK_GBS / 1e3)
        ops = ug_amd.LlamaOps.hip()
        cm = ops.custom_softmax(src)
        cs2 = Schedule.create_one(cm).compile()
        _, ms = timed(dev, cs2.run, steps, warmup)
        gbs = 8.0 * rows * cols * steps / (ms * 1e-3) / 1e9
        out[f"softmax_custom_{rows}x{cols}"] = {"GB/s": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4), "us_per_softmax": round(ms * 1e3 / steps, 2),
                                               "launches": 1}
        if rows * cols * 8 < (1 << 22):
            out[f"softmax_custom_{rows}x{cols}"]["bound"] = "1 launch floor"
    return out


def check_product_rows(name, got, a, w, k, bf16, rows=(0, 1, 255, 256, 511, 777, 1023)):
    """Rows of a product read back from the device against the float64 product of the same rows: within the forward
    bound of an f32 summation (k eps sum|a||b|), plus one rounding to bf16 (2^-8) when the result is stored as bf16.
    got, a: [b, m, *]; w: [b, k, n].  Raises when the device result is off: nothing unverified is timed."""
    eps = float(np.finfo(np.float32).eps)
    rows = [r for r in rows if r < a.shape[1]]
    a64, w64 = a[:, rows].astype(np.float64), w.astype(np.float64)
    exact = np.matmul(a64, w64)
    bound = k * eps * np.matmul(np.abs(a64), np.abs(w64)) + (2.0 ** -8 * np.abs(exact) if bf16 else 0.0)
    err = np.abs(got[:, rows].astype(np.float64) - exact)
    if not np.all(err <= bound * 1.001 + 1e-12):
        raise RuntimeError(f"{name}: device result outside the f64 bound on rows {rows} (max error {err.max():.3g}, bound there {bound.flat[int(err.argmax())]:.3g})")
    return {"rows_checked": len(rows) * a.shape[0], "max_abs_err": float(err.max()), "max_err_over_bound": float((err / (bound + 1e-300)).max())}


# What one launch of the 8 x 1024^3 bf16 product cannot go below on this chip, from figures measured with the lab kernels of
# the `floors` group and with ablated builds of the GEMM (null kernel with the same grid and LDS: 2.3 us between dependent
# launches; first K tile's trip to memory: 0.7 us; 16 MiB stored by 256 CUs at once: 1.7 us past the cache, 2.4 through it;
# nothing but bf16 MFMAs on U(-1, 1) operands: 1.80-1.83 PFLOP/s, the chip's power limit).  One round of 256 workgroups: none
# of the four overlaps another.
def bmm_bf16_bound_us(flop, operand_and_result_bytes, launch_us=2.3, first_tile_us=0.7, store_us=1.7, mfma_power_limited_tf=1815.0, stream_gbs=6400.0):
    mfma = flop / mfma_power_limited_tf / 1e6
    return {"launch": launch_us, "first_tile": first_tile_us, "mfma_at_the_power_limited_rate": round(mfma, 2), "result_store": store_us,
            "sum": round(launch_us + first_tile_us + mfma + store_us, 2),
            "hbm_only": round(operand_and_result_bytes / stream_gbs / 1e3 + launch_us, 2),
            "note": "sum = launch + first tile + flop / 1.815 PFLOP/s (MFMA-only kernel, random operands) + result store; hbm_only = 48 MiB at 6.4 TB/s + launch"}


def bmm(dev, steps, warmup):
    """Config 3: batched matmul 8 x 1024^3, f32 through the lazy graph and bf16 through Device::matmul.  Every product
    is read back and sampled rows are checked against float64 before it is timed."""
    import ug_amd
    from ug_amd import LazyBuffer as LB, Schedule, rng
    out = {}
    b, m = 8, 1024
    flop = 2.0 * b * m * m * m
    a = rng.uniform_pm1(4, b * m * m)
    w = rng.uniform_pm1(5, b * m * m)
    la, lw = LB.copy(a, (b, m, m), dev), LB.copy(w, (b, m, m), dev)
    mm = la.matmul(lw)
    cs = Schedule.create_one(mm).compile()
    cs.run()
    chk = check_product_rows("bmm_f32", mm.data_vec().reshape(b, m, m), a.reshape(b, m, m), w.reshape(b, m, m), m, False)
    kernel = ug_amd.last_kernel()
    _, ms = timed_hot(dev, cs.run, steps, warmup)
    tf = flop * steps / (ms * 1e-3) / 1e12
    out["bmm_f32_8x1024^3"] = {"TFLOP/s": round(tf, 2), "frac_mfma_f32": round(tf / MFMA_F32_PEAK_TF, 4), "us": round(ms * 1e3 / steps, 1), "kernel": kernel, "verified": chk}
    # the same product, and a large one, as six bf16 terms on the bf16 matrix pipe (UGHIP_MATMUL_X6=1, opt-in: the f32
    # product's accuracy, not its bits): the rate is that of the f32 product it stands for, frac_mfma_bf16 counts 6 x the flops
    with ug_amd.tuning(MATMUL_X6=1):
        cs.run()
        chk = check_product_rows("bmm_f32_x6", mm.data_vec().reshape(b, m, m), a.reshape(b, m, m), w.reshape(b, m, m), m, False)
        kernel = ug_amd.last_kernel()
        _, ms = timed_hot(dev, cs.run, steps, warmup)
    tf = flop * steps / (ms * 1e-3) / 1e12
    out["bmm_f32_8x1024^3_six_bf16_terms"] = {"TFLOP/s_f32_equivalent": round(tf, 2), "times_the_f32_matrix_peak": round(tf / MFMA_F32_PEAK_TF, 3), "frac_mfma_bf16": round(6 * tf / MFMA_BF16_PEAK_TF, 4),
                                              "us": round(ms * 1e3 / steps, 1), "kernel": kernel, "verified": chk}
    m4 = 4096
    a4, w4 = rng.uniform_pm1(4, m4 * m4), rng.uniform_pm1(5, m4 * m4)
    mm4 = LB.copy(a4, (1, m4, m4), dev).matmul(LB.copy(w4, (1, m4, m4), dev))
    cs4 = Schedule.create_one(mm4).compile()
    for key, sw_ in (("mm_f32_nn_4096^3", {}), ("mm_f32_nn_4096^3_six_bf16_terms", {"MATMUL_X6": 1})):
        with ug_amd.tuning(**sw_):
            cs4.run()
            chk = check_product_rows(key, mm4.data_vec().reshape(1, m4, m4), a4.reshape(1, m4, m4), w4.reshape(1, m4, m4), m4, False)
            kernel = ug_amd.last_kernel()
            _, ms = timed_hot(dev, cs4.run, max(5, steps // 4), 2)
        tf = 2.0 * m4 ** 3 * max(5, steps // 4) / (ms * 1e-3) / 1e12
        row = {"us": round(ms * 1e3 / max(5, steps // 4), 1), "kernel": kernel, "verified": chk}
        row["TFLOP/s_f32_equivalent" if sw_ else "TFLOP/s"] = round(tf, 2)
        if sw_:
            row["times_the_f32_matrix_peak"], row["frac_mfma_bf16"] = round(tf / MFMA_F32_PEAK_TF, 3), round(6 * tf / MFMA_BF16_PEAK_TF, 4)
        else:
            row["frac_mfma_f32"] = round(tf / MFMA_F32_PEAK_TF, 4)
        out[key] = row
    del mm4, cs4
    ab, wb = rng.bf16_round(a), rng.bf16_round(w)
    sa, sw = dev.slice_from(rng.to_bf16_bits(a)), dev.slice_from(rng.to_bf16_bits(w))
    dst = dev.allocate_uninit(ug_amd.BF16, b * m * m)
    lay = ((b, m, m), (m * m, m, 1), 0)
    run = lambda: dev.matmul(dst, sa, sw, (b, m, m, m), lay, lay)  # noqa: E731
    run()
    chk = check_product_rows("bmm_bf16", rng.from_bf16_bits(dst.to_vec()).reshape(b, m, m), ab.reshape(b, m, m), wb.reshape(b, m, m), m, True)
    kernel = ug_amd.last_kernel()
    _, ms = timed_hot(dev, run, steps, warmup)
    tf = flop * steps / (ms * 1e-3) / 1e12
    out["bmm_bf16_8x1024^3"] = {"TFLOP/s": round(tf, 2), "frac_mfma_bf16": round(tf / MFMA_BF16_PEAK_TF, 4), "us": round(ms * 1e3 / steps, 1), "kernel": kernel, "verified": chk,
                                "bound_us": bmm_bf16_bound_us(flop, 3 * 2 * b * m * m)}
    # large products, the rhs stored [n, k] (what matmul_t of the llama projections hands over) and row-major
    m = 4096
    a, w = rng.uniform_pm1(4, m * m), rng.uniform_pm1(5, m * m)
    ab, wb = rng.bf16_round(a).reshape(1, m, m), rng.bf16_round(w).reshape(1, m, m)
    sa, sw = dev.slice_from(rng.to_bf16_bits(a)), dev.slice_from(rng.to_bf16_bits(w))
    dst = dev.allocate_uninit(ug_amd.BF16, m * m)
    for key, rhs_l, w_kn in (("mm_bf16_nt_4096^3", ((1, m, m), (m * m, 1, m), 0), np.swapaxes(wb, 1, 2)), ("mm_bf16_nn_4096^3", ((1, m, m), (m * m, m, 1), 0), wb)):
        run = lambda: dev.matmul(dst, sa, sw, (1, m, m, m), ((1, m, m), (m * m, m, 1), 0), rhs_l)  # noqa: E731
        run()
        chk = check_product_rows(key, rng.from_bf16_bits(dst.to_vec()).reshape(1, m, m), ab, w_kn, m, True, rows=(0, 255, 256, 2049, 4095))
        kernel = ug_amd.last_kernel()
        _, ms = timed_hot(dev, run, steps, warmup)
        tf = 2.0 * m * m * m * steps / (ms * 1e-3) / 1e12
        out[key] = {"TFLOP/s": round(tf, 2), "frac_mfma_bf16": round(tf / MFMA_BF16_PEAK_TF, 4), "us": round(ms * 1e3 / steps, 1), "kernel": kernel, "verified": chk}
    # rows the 256-row tiles do not divide (a prompt of 3000 tokens against a 4096 x 4096 matrix): the same kernel, its last tiles hang over the end
    mr, nr = 3000, 4096
    a, w = rng.uniform_pm1(4, mr * nr), rng.uniform_pm1(5, nr * nr)
    ab, wb = rng.bf16_round(a).reshape(1, mr, nr), rng.bf16_round(w).reshape(1, nr, nr)
    sa, sw = dev.slice_from(rng.to_bf16_bits(a)), dev.slice_from(rng.to_bf16_bits(w))
    dst = dev.allocate_uninit(ug_amd.BF16, mr * nr)
    run = lambda: dev.matmul(dst, sa, sw, (1, mr, nr, nr), ((1, mr, nr), (mr * nr, nr, 1), 0), ((1, nr, nr), (nr * nr, 1, nr), 0))  # noqa: E731
    run()
    chk = check_product_rows("mm_bf16_nt_3000x4096x4096", rng.from_bf16_bits(dst.to_vec()).reshape(1, mr, nr), ab, np.swapaxes(wb, 1, 2), nr, True, rows=(0, 255, 256, 2815, 2816, 2999))
    kernel = ug_amd.last_kernel()
    _, ms = timed_hot(dev, run, steps, warmup)
    tf = 2.0 * mr * nr * nr * steps / (ms * 1e-3) / 1e12
    out["mm_bf16_nt_3000x4096x4096"] = {"TFLOP/s": round(tf, 2), "frac_mfma_bf16": round(tf / MFMA_BF16_PEAK_TF, 4), "us": round(ms * 1e3 / steps, 1), "kernel": kernel, "verified": chk}
    del sa, sw, dst
    # the same kernel where the fixed cost (launch, first tile, the result's way out: ~9 us) is 1 % of the run
    m = 8192
    a, w = rng.uniform_pm1(4, m * m), rng.uniform_pm1(5, m * m)
    ab, wb = rng.bf16_round(a).reshape(1, m, m), rng.bf16_round(w).reshape(1, m, m)
    sa, sw = dev.slice_from(rng.to_bf16_bits(a)), dev.slice_from(rng.to_bf16_bits(w))
    dst = dev.allocate_uninit(ug_amd.BF16, m * m)
    run = lambda: dev.matmul(dst, sa, sw, (1, m, m, m), ((1, m, m), (m * m, m, 1), 0), ((1, m, m), (m * m, 1, m), 0))  # noqa: E731
    run()
    chk = check_product_rows("mm_bf16_nt_8192^3", rng.from_bf16_bits(dst.to_vec()).reshape(1, m, m), ab, np.swapaxes(wb, 1, 2), m, True, rows=(0, 257, 4097, 8191))
    kernel = ug_amd.last_kernel()
    _, ms = timed_hot(dev, run, 20, 3)
    tf = 2.0 * m * m * m * 20 / (ms * 1e-3) / 1e12
    out["mm_bf16_nt_8192^3"] = {"TFLOP/s": round(tf, 2), "frac_mfma_bf16": round(tf / MFMA_BF16_PEAK_TF, 4), "us": round(ms * 1e3 / 20, 1), "kernel": kernel, "verified": chk}
    del sa, sw, dst
    # The products of a 128-token prompt (f32 rows against bf16 matrices stored [n, k]): the f32 matrix pipe on the widened
    # matrix against three bf16 terms per row element on the bf16 pipe.  TFLOP/s counts 2 m n k either way.  The same matrix
    # every step: up to 131 MB that stay in the 256 MB memory-side cache; inside a model every layer's matrices come from HBM
    # and the same kernels take 1-2 us longer (the llama rows' prefill_ms_warm has that).
    t = 128
    for label, n, k in (("qkv", 2560, 2048), ("gate_up", 11264, 2048), ("down", 2048, 5632), ("head", 32000, 2048)):
        xh = rng.normal(21, t * k)
        wh = rng.bf16_round(rng.normal(22, n * k, 0.05))
        x, w = LB.copy(xh, (1, t, k), dev), LB.copy(rng.to_bf16_bits(wh), (n, k), dev)
        for name, ops in (("f32_pipe", ug_amd.LlamaOps.hip()), ("bf16x3", ug_amd.LlamaOps.hip(bf16x3=True))):
            key = f"prefill_{label}_128x{n}x{k}_{name}"
            lb = ops.linear(x, w)
            cs = Schedule.create_one(lb).compile()
            cs.run()
            kernel = ug_amd.last_kernel()
            chk = check_product_rows(key, lb.data_vec().reshape(1, t, n), xh.reshape(1, t, k), np.swapaxes(wh.reshape(1, n, k), 1, 2), k, False, rows=(0, 1, 63, 64, 127))
            _, ms = timed_hot(dev, cs.run, steps, warmup, 0.1)
            tf = 2.0 * t * n * k * steps / (ms * 1e-3) / 1e12
            if name == "bf16x3":   # three bf16 MFMA products per element product: the pipe that does the work is the bf16 one
                out[key] = {"TFLOP/s_f32_equivalent": round(tf, 2), "TFLOP/s_on_the_bf16_pipe": round(3 * tf, 2), "frac_mfma_bf16": round(3 * tf / MFMA_BF16_PEAK_TF, 4),
                            "us": round(ms * 1e3 / steps, 1), "kernel": kernel, "verified": chk}
            else:
                out[key] = {"TFLOP/s": round(tf, 2), "frac_mfma_f32": round(tf / MFMA_F32_PEAK_TF, 4), "us": round(ms * 1e3 / steps, 1), "kernel": kernel, "verified": chk}
    return out


def verify(name, got, want, rtol=1e-5, atol=1e-30):
    """Raises unless got == want within rtol / atol: every extra checks its device output before it is timed."""
    got, want = np.asarray(got, np.float64).reshape(-1), np.asarray(want, np.float64).reshape(-1)
    bad = ~(np.abs(got - want) <= atol + rtol * np.abs(want))
    if got.shape != want.shape or bad.any():
        i = int(np.argmax(bad))
        raise RuntimeError(f"{name}: device output differs from the float64 statement at {int(bad.sum())} of {want.size} elements (first: [{i}] {got[i]} vs {want[i]})")
    return True


def softmax64(x):
    x = np.asarray(x, np.float64)
    e = np.exp(x - x.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


def llama_pieces(dev, steps, warmup):
    """Config 4: the llama layer pieces at T=512, hidden 2048, 32 heads x 64 (f32), each as the lazy
    graph ug-llama builds for it (ug-llama/src/model.rs:32-109,203-248), with its algorithmic bytes.  Each piece's
    output is checked against a float64 numpy statement before it is timed."""
    import ug_amd
    from ug_amd import LazyBuffer as LB, Schedule, rng
    ll, ops = ug_amd.llama, ug_amd.LlamaOps.hip()
    out = {}
    t, hidden, heads, hd = 512, 2048, 32, 64

    def hbm(name, lb, nbytes, want=None, rtol=1e-5, atol=1e-30):
        cs = Schedule.create_one(lb).compile()
        cs.run()
        ok = verify(name, lb.data_vec(), want() if callable(want) else want, rtol, atol) if want is not None else False
        _, ms = timed(dev, cs.run, steps, warmup)
        gbs = nbytes * steps / (ms * 1e-3) / 1e9
        out[name] = {"GB/s": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4), "us": round(ms * 1e3 / steps, 2), "algorithmic_bytes": nbytes, "verified": ok}
        if gbs > HBM_PEAK_GBS:
            # a working set of a few tens of MB lives in the caches (32 MB of L2, 256 MB memory-side): the rate is theirs, and a
            # fraction of the HBM peak says nothing; the same kernel on a 1 GiB working set is under `hbm_large`
            out[name]["frac_hbm"] = None
            out[name]["note"] = "cache-resident working set: faster than HBM's peak, no HBM fraction quoted"

    xh, ah = rng.normal(6, t * hidden).reshape(1, t, hidden), rng.normal(6 + 100, hidden, 0.02)
    x = LB.copy(xh, (1, t, hidden), dev)
    alpha = LB.copy(ah, (hidden,), dev)
    x64 = xh.astype(np.float64)
    hbm("c4_rms_norm_512x2048", ll.rms_norm(x, alpha, 1e-5), 2 * 4 * t * hidden + 4 * hidden,
        x64 / np.sqrt((x64 * x64).mean(-1, keepdims=True) + np.float64(np.float32(1e-5))) * ah.astype(np.float64), atol=1e-9)
    cfg = ug_amd.LlamaConfig()
    cos, sin = ll.rope_tables(dev, cfg)
    cos.realize()   # the tables are built once per model (ug-llama/src/model.rs:147-168), not per layer call
    sin.realize()
    qh = rng.normal(7, heads * t * hd).reshape(1, heads, t, hd)
    q = LB.copy(qh, (1, heads, t, hd), dev)
    pos = LB.copy(np.zeros(1, np.int32), (1,), dev)
    c64, s64 = cos.data_vec().reshape(-1, hd // 2)[:t].astype(np.float64), sin.data_vec().reshape(-1, hd // 2)[:t].astype(np.float64)
    q1, q2 = qh[..., :hd // 2].astype(np.float64), qh[..., hd // 2:].astype(np.float64)
    hbm("c4_rope_q_1x32x512x64", ops.rope(q, cos, sin, pos), 2 * 4 * heads * t * hd + 2 * 4 * t * (hd // 2),
        np.concatenate([q1 * c64 - q2 * s64, q1 * s64 + q2 * c64], -1), rtol=0, atol=4 * float(np.finfo(np.float32).eps) * float(np.abs(qh).max()))
    sh = rng.normal(8, heads * t * t).reshape(1, heads, t, t)
    s = LB.copy(sh, (1, heads, t, t), dev)
    keep = np.arange(t)[None, :] <= np.arange(t)[:, None]
    masked = np.where(keep, sh, np.float32(-np.inf))
    plain, causal = softmax64(sh), softmax64(masked)
    # the mask is exact (-inf where i2 > i1): compared bit for bit rather than through the tolerance helper
    mk = ops.causal_mask(s)
    if not np.array_equal(mk.data_vec().reshape(sh.shape), masked):
        raise RuntimeError("c4_causal_mask: device output differs from the mask")
    # bytes: the kept triangle is read, every element is written (the masked half is -inf whatever it held); the reference's
    # CPU op reads everything (2 x 4 B per element), kept beside it as the reference's formula
    mask_bytes = 4 * heads * (t * (t + 1) // 2 + t * t)
    hbm("c4_causal_mask_1x32x512x512", ops.causal_mask(s), mask_bytes)   # a fresh node: mk is realised and would schedule nothing
    out["c4_causal_mask_1x32x512x512"].update({"verified": True, "bytes_reading_everything": 2 * 4 * heads * t * t,
                                                "note": "algorithmic bytes = kept triangle read + full write; cache-resident at this size"})
    hbm("c4_softmax_lazy_1x32x512x512", ll.softmax(s), 2 * 4 * heads * t * t, plain)
    hbm("c4_softmax_custom_1x32x512x512", ops.custom_softmax(s), 2 * 4 * heads * t * t, plain)
    hbm("c4_mask_then_softmax_custom", ops.custom_softmax(ops.causal_mask(s)), mask_bytes + 2 * 4 * heads * t * t, causal)
    # the same two ops as one kernel: reads the kept triangle, writes every element
    hbm("c4_causal_softmax_fused", ops.causal_softmax(s), mask_bytes, causal)
    gh, uh = rng.normal(8 + 100, t * 5632), rng.normal(8 + 101, t * 5632)
    gate = LB.copy(gh, (1, t, 5632), dev)
    up = LB.copy(uh, (1, t, 5632), dev)
    g64 = gh.astype(np.float64)
    hbm("c4_silu_mul_512x5632", ll.silu(gate).binary("mul", up), 3 * 4 * t * 5632, g64 / (1.0 + np.exp(-g64)) * uh.astype(np.float64), atol=1e-9)

    def gemm(name, lhs, rhs, transposed, b, m, n, k, a_h, w_kn):
        mm = lhs.matmul_t(rhs) if transposed else lhs.matmul(rhs)
        cs = Schedule.create_one(mm).compile()
        cs.run()
        chk = check_product_rows(name, mm.data_vec().reshape(b, m, n), a_h.reshape(b, m, k), w_kn.reshape(b, k, n), k, False, rows=(0, 1, 255, 256, 511))
        kernel = ug_amd.last_kernel()
        _, ms = timed_hot(dev, cs.run, steps, warmup, 0.1)
        flop, nbytes = 2.0 * b * m * n * k, 4.0 * b * (m * k + k * n + m * n)
        sec = ms * 1e-3 / steps
        out[name] = {"TFLOP/s": round(flop / sec / 1e12, 2), "frac_mfma_f32": round(flop / sec / 1e12 / MFMA_F32_PEAK_TF, 4), "GB/s": round(nbytes / sec / 1e9, 1),
                     "frac_hbm": round(nbytes / sec / 1e9 / HBM_PEAK_GBS, 4), "us": round(sec * 1e6, 2), "kernel": kernel, "verified": chk}

    kh, vh = rng.normal(8 + 200, heads * t * hd).reshape(1, heads, t, hd), rng.normal(8 + 300, heads * t * hd).reshape(1, heads, t, hd)
    kk = LB.copy(kh, (1, heads, t, hd), dev)
    v = LB.copy(vh, (1, heads, t, hd), dev)
    gemm("c4_qk_t_b32_512x512x64", q, kk, True, heads, t, t, hd, qh, np.ascontiguousarray(np.swapaxes(kh, -1, -2)))
    gemm("c4_att_v_b32_512x64x512", s, v, False, heads, t, hd, t, sh, vh)

    # the whole chain either side of the softmax (rope(q), repeat, q k^T, scale, mask, softmax, x v, transposes) as one
    # kernel over preallocated caches of 4 kv heads: scores stay in registers.  flop = the two causal products.
    nkv, cap = 4, 2048
    qfh = rng.normal(7, t * heads * hd).reshape(1, t, heads * hd)
    kch, vch = rng.normal(8 + 200, nkv * cap * hd).reshape(1, nkv, cap, hd), rng.normal(8 + 300, nkv * cap * hd).reshape(1, nkv, cap, hd)
    qf = LB.copy(qfh, (1, t, heads * hd), dev)
    kc = LB.copy(kch, (1, nkv, cap, hd), dev)
    vc = LB.copy(vch, (1, nkv, cap, hd), dev)
    scale = float(np.float32(hd) ** np.float32(-0.5))
    att = ops.attention_cached(qf, kc, vc, t, scale, cos, sin, pos, False)
    cs = Schedule.create_one(att).compile()
    cs.run()
    got = att.data_vec().reshape(t, heads, hd)
    for h in (0, 13, 31):     # three of the 32 heads against float64 causal attention (keys as cached: not rotated again)
        qq = qfh.reshape(t, heads, hd)[:, h].astype(np.float64)
        qr = np.concatenate([qq[:, :hd // 2] * c64 - qq[:, hd // 2:] * s64, qq[:, :hd // 2] * s64 + qq[:, hd // 2:] * c64], -1)
        kv = h // (heads // nkv)
        p = softmax64(np.where(keep, qr @ kch[0, kv, :t].astype(np.float64).T * scale, -np.inf))
        verify(f"c4_attention_cached head {h}", got[:, h], p @ vch[0, kv, :t].astype(np.float64), rtol=0, atol=2e-5 * float(np.abs(got).max()))
    _, ms = timed_hot(dev, cs.run, steps, warmup, 0.1)
    sec = ms * 1e-3 / steps
    flop = 2 * 2.0 * heads * hd * t * (t + 1) / 2
    nbytes = 4.0 * (2 * t * heads * hd + 2 * nkv * t * hd)
    # 256 positions and up take both products as six bf16 terms on the bf16 matrix pipe (the f32 MFMAs of the other kernel
    # occupy the vector ALU): TFLOP/s and frac_mfma_f32 are the f32 products the op stands for against the f32 peak,
    # frac_mfma_bf16 prices the six-fold flops it actually issues against the bf16 peak.
    out["c4_attention_cached_t512"] = {"us": round(sec * 1e6, 2), "TFLOP/s": round(flop / sec / 1e12, 2), "frac_mfma_f32": round(flop / sec / 1e12 / MFMA_F32_PEAK_TF, 4),
                                       "frac_mfma_bf16": round(6 * flop / sec / 1e12 / MFMA_BF16_PEAK_TF, 4), "kernel": "att_planes_kernel + attention_prefill_x6_kernel<2>",
                                       "algorithmic_bytes": int(nbytes), "verified": True,
                                       "replaces": "c4_rope_q + c4_qk_t + c4_causal_softmax_fused + c4_att_v + 2 repeats + 2 transposes"}
    # the same op over a prompt of 2048 positions (a full cache), and with the f32 products it had before
    t2 = cap
    q2h = rng.normal(17, t2 * heads * hd).reshape(1, t2, heads * hd)
    q2 = LB.copy(q2h, (1, t2, heads * hd), dev)
    flop2 = 2 * 2.0 * heads * hd * t2 * (t2 + 1) / 2
    for name, x6 in (("attention_cached_t2048", None), ("attention_cached_t2048_f32_products", 0)):
        with (ug_amd.tuning(ATT_X6=x6) if x6 is not None else contextlib.nullcontext()):
            att2 = ops.attention_cached(q2, kc, vc, t2, scale)
            cs2 = Schedule.create_one(att2).compile()
            cs2.run()
            got2 = att2.data_vec().reshape(t2, heads, hd)
            for h in (5, 30):     # two heads, the last 64 positions against float64
                kv = h // (heads // nkv)
                qq = q2h.reshape(t2, heads, hd)[-64:, h].astype(np.float64)
                sc = qq @ kch[0, kv, :t2].astype(np.float64).T * scale
                sc = np.where(np.arange(t2)[None, :] <= (t2 - 64 + np.arange(64))[:, None], sc, -np.inf)
                verify(f"{name} head {h}", got2[-64:, h], softmax64(sc) @ vch[0, kv, :t2].astype(np.float64), rtol=0, atol=2e-5 * float(np.abs(got2).max()))
            _, ms = timed_hot(dev, cs2.run, max(10, steps // 4), warmup, 0.1)
        sec = ms * 1e-3 / max(10, steps // 4)
        out[name] = {"us": round(sec * 1e6, 2), "TFLOP/s": round(flop2 / sec / 1e12, 2), "frac_mfma_f32": round(flop2 / sec / 1e12 / MFMA_F32_PEAK_TF, 4), "verified": True}
        if x6 is None:
            out[name]["frac_mfma_bf16"] = round(6 * flop2 / sec / 1e12 / MFMA_BF16_PEAK_TF, 4)
    return out


def hbm_large(dev, steps, warmup):
    """The memory-bound kernels on working sets the 256 MB Infinity Cache cannot hold (1 GiB each), next to the BASELINE
    sizes above: what the same lowered kernels sustain from HBM proper."""
    import ug_amd
    from ug_amd import LazyBuffer as LB, Schedule, rng
    ll, ops = ug_amd.llama, ug_amd.LlamaOps.hip()
    out = {}
    steps = max(10, steps // 4)

    def tile(seed, n, std=None):
        base = rng.uniform_pm1(seed, 1 << 22) if std is None else rng.normal(seed, 1 << 22, std)
        return np.tile(base, n >> 22)

    def hbm(name, lb, nbytes, check):
        cs = Schedule.create_one(lb).compile()
        cs.run()
        check(lb)
        _, ms = timed(dev, cs.run, steps, min(warmup, 5))
        gbs = nbytes * steps / (ms * 1e-3) / 1e9
        out[name] = {"GB/s": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4), "us": round(ms * 1e3 / steps, 1), "algorithmic_bytes": nbytes,
                     "working_set_MiB": nbytes >> 20, "verified": True}

    # config 2's graph at 2^27 elements: 2 x 512 MiB read
    n = 1 << 27
    a, b = tile(2, n), tile(3, n)
    truth = float(np.sum(a.astype(np.float64) * b + 0.5 * a.astype(np.float64)))
    from ug_amd.graphs import fused_reduce_graph
    la, lb_ = LB.copy(a, (n,), dev), LB.copy(b, (n,), dev)

    def chk_sum(r):
        got = float(r.data_vec()[0])
        if not abs(got - truth) <= 1e-5 * abs(truth) + 1e-1:
            raise RuntimeError(f"fused_reduce_2pow27: {got} vs {truth}")
    hbm("fused_reduce_2pow27", fused_reduce_graph(la, lb_, dev), 2 * 4 * n + 4, chk_sum)
    del la, lb_, a, b
    # softmax over 32768 x 4096 f32: 512 MiB read, 512 MiB written (8 B per element, the reference's formula)
    rows, cols = 32768, 4096
    xh = tile(1, rows * cols, 3.0).reshape(rows, cols)
    want_rows = softmax64(xh[[0, 1, 1023, 20000, rows - 1]])

    def chk_sm(r):
        got = r.data_vec().reshape(rows, cols)[[0, 1, 1023, 20000, rows - 1]]
        verify("softmax_32768x4096", got, want_rows)
    x = LB.copy(xh, (rows, cols), dev)
    hbm("softmax_custom_32768x4096", ops.custom_softmax(x), 8 * rows * cols, chk_sm)
    hbm("softmax_lazy_32768x4096", ll.softmax(x), 8 * rows * cols, chk_sm)
    # causal mask over [1, 128, 1024, 1024]: 512 MiB in, 512 MiB out
    sh = xh.reshape(1, 128, 1024, 1024)
    keep = np.arange(1024)[None, :] <= np.arange(1024)[:, None]

    def chk_mask(r):
        got = r.data_vec().reshape(sh.shape)[0, [0, 77, 127]]
        if not np.array_equal(got, np.where(keep, sh[0, [0, 77, 127]], np.float32(-np.inf))):
            raise RuntimeError("causal_mask_1x128x1024x1024: device output differs from the mask")
    s = LB.copy(sh, sh.shape, dev)
    hbm("causal_mask_1x128x1024x1024", ops.causal_mask(s), 4 * 128 * (1024 * 1025 // 2 + 1024 * 1024), chk_mask)   # kept triangle read + full write
    out["causal_mask_1x128x1024x1024"]["bytes_reading_everything"] = 8 * rows * cols
    del s, x
    # SwiGLU over [16384, 5632] f32: 2 x 352 MiB read, 352 MiB written
    t, f = 16384, 5632
    gh, uh = tile(108, t * f, 1.0), tile(109, t * f, 1.0)
    g64 = gh[:4096].astype(np.float64)
    want = g64 / (1.0 + np.exp(-g64)) * uh[:4096].astype(np.float64)

    def chk_silu(r):
        verify("silu_mul_16384x5632", r.data_vec()[:4096], want, atol=1e-9)
    hbm("silu_mul_16384x5632", ll.silu(LB.copy(gh, (1, t, f), dev)).binary("mul", LB.copy(uh, (1, t, f), dev)), 3 * 4 * t * f, chk_silu)
    return out


def config5_ids_check(toks, st, n_prompt, n_steps, bf16_rounded, norm_mean=0.0):
    """The ids of the timed run against what the CPU oracle wrote for BASELINE config 5 (tests/golden/llama_config5*_greedy.json,
    made by tests/golden/make_llama_config5_fixture.py): every id up to the first position where the oracle's own top-1
    margin is inside the tie band must be equal, or the run is reported as failed.  Three fixtures: BASELINE's weights
    (128 + 128 positions; logits within 1e-4 of each other, a two-cycle of ids), the same model with norm vectors 1 + N(0, 0.02)
    (128 + 128: logits of 3 to 5, 113 distinct ids), and that model behind a prompt of 1900 tokens (+ 64)."""
    name, tie, top_tol = "llama_config5_greedy.json", 4e-5, 2e-5
    if norm_mean == 1.0:
        name, tie, top_tol = ("llama_config5_unit_norms_prompt1900_greedy.json" if n_prompt == 1900 else "llama_config5_unit_norms_greedy.json"), 4e-4, 2e-4
    elif norm_mean != 0.0:
        return {"checked": False, "why": "no fixture for these weights"}
    path = os.path.join(ROOT, "tests", "golden", name)
    if not os.path.exists(path):
        return {"checked": False, "why": "fixture missing"}
    with open(path) as f:
        fx = json.load(f)
    if n_prompt != fx["prompt"]["n"] or n_steps != fx["steps"]:
        return {"checked": False, "why": f"the fixture holds {fx['prompt']['n']} + {fx['steps']} positions"}
    run = fx["runs"]["bf16_rounded" if bf16_rounded else "f32"]
    ids_o, mar_o, top_o = np.array(run["ids"]), np.array(run["margin"]), np.array(run["top1"])
    diff = np.flatnonzero(np.asarray(toks) != ids_o)
    first = int(diff[0]) if diff.size else None
    if first is not None and mar_o[first] > tie:
        raise RuntimeError(f"llama ids part from the oracle's at position {first} where its margin is {mar_o[first]:.3g}")
    upto = first if first is not None else ids_o.size
    top_err = float(np.abs(np.asarray(st["top1"])[:upto] - top_o[:upto]).max()) if upto else 0.0
    if top_err > top_tol:
        raise RuntimeError(f"llama top logits differ from the oracle's by {top_err:.3g}")
    return {"checked": True, "fixture": name, "ids_equal": int(ids_o.size - diff.size), "of": int(ids_o.size), "distinct_ids": len(set(ids_o.tolist())), "first_difference": first,
            "max_abs_top1_diff": top_err, "tie_band": tie, "positions_outside_tie_band": int((mar_o > tie).sum())}


def llama_decode(dev, n_prompt=128, n_steps=128, fused_attention=0, bf16_matrices=False, bf16x3=False, norm_mean=0.0):
    """Config 5: TinyLlama-1.1B shape, random-init f32 weights, prefill 128 then 128 greedy steps.
    Fresh buffers are not zero-filled here (every kernel of the model writes its whole output; the
    ids are the same either way, which the GPU tests check).  fused_attention: 0 = the reference's
    op-by-op graph; 1 = ughip_causal_softmax_rows / ughip_rope_append / ughip_attention_decode;
    2 = caches written in place (ughip_kv_append) and ughip_attention_cached for prefill and decode;
    3 = 2 plus packed q|k|v, gate/up + SwiGLU and residual projections (ughip_gemv_multi / _gate_up / _add).
    bf16_matrices: bf16-rounded weights, the projection matrices and the head kept and streamed as bf16
    (activations, caches, norms f32): the numbers of the f32 model on the rounded weights from half the bytes.
    bf16x3: with bf16 matrices, products over nine or more rows (the prompt) split every row element into three bf16
    terms and run on the bf16 matrix pipe (UGHIP_PRODUCT_BF16X3): exact product terms, f32 sums in another order.
    norm_mean: the norm vectors are norm_mean + N(0, 0.02) (BASELINE: 0; 1 is what checkpoints hold and what gives ids that
    carry information -- same kernels, same bytes, same time)."""
    import ug_amd
    from ug_amd import rng
    cfg = ug_amd.LlamaConfig()
    ops = ug_amd.LlamaOps.hip(bf16x3=bf16x3)
    dev.set_zero_fill(False)
    t0 = time.perf_counter()
    model = ug_amd.LlamaModel(dev, ops, cfg, custom_softmax=True, seed=9, std=0.02, round_bf16=bf16_matrices, fused_attention=fused_attention,
                              bf16_matrices=bf16_matrices, norm_mean=norm_mean)
    load_s = time.perf_counter() - t0
    prompt = rng.token_ids(10, n_prompt, cfg.vocab_size)
    model.generate(prompt, 4)          # compiles every kernel shape family once
    toks, st = model.generate(prompt, n_steps)
    # the same prompt eight more times back to back: what a prefill costs once the chip is at its working clocks (the
    # first one above comes behind host work and a handful of short launches)
    warm_ms = round(min(model.generate(prompt, 0)[1]["prefill_ms"] for _ in range(8)), 2) if fused_attention == 3 else None
    # what a prompt of another length costs (level 3 with bf16 matrices only: short prompts take 32- and 64-row tiles)
    by_length = {}
    if fused_attention == 3 and bf16_matrices and n_prompt == 128:
        for t in (2, 16, 64, 512):
            p_t = rng.token_ids(10, t, cfg.vocab_size)
            model.generate(p_t, 1)
            by_length[str(t)] = round(min(model.generate(p_t, 0)[1]["prefill_ms"] for _ in range(3)), 2)
    dev.set_zero_fill(True)
    check = config5_ids_check(toks, st, n_prompt, n_steps, bf16_matrices, norm_mean)
    # streamed per token: every matrix once (2 or 4 bytes per weight); the 45 norm vectors stay f32
    weights_bytes = (2 if bf16_matrices else 4) * 1034512384
    tok_s = n_steps / (st["decode_ms"] * 1e-3)
    return {"tok/s": round(tok_s, 2), "decode_ms_per_token": round(st["decode_ms"] / n_steps, 3), "prefill_ms": round(st["prefill_ms"], 1),
            "frac_hbm_weights_only": round(tok_s * weights_bytes / 1e9 / HBM_PEAK_GBS, 4), "load_s": round(load_s, 1), "dtype": "f32 activations, bf16 matrices" if bf16_matrices else "f32", "zero_fill": False, "fused_attention": fused_attention, "norm_vectors": "N(0, 0.02) (BASELINE)" if norm_mean == 0.0 else f"{norm_mean:g} + N(0, 0.02)",
            "launches_per_token": st.get("decode_items"), "prefill_product": "bf16x3" if bf16x3 else "f32", "prompt_tokens": n_prompt, "decode_steps": n_steps, "first_ids": toks[:8].tolist(), "min_top1_margin": float(st["margins"].min()), "ids_vs_oracle_fixture": check,
            **({"prefill_ms_warm": warm_ms} if warm_ms is not None else {}), **({"prefill_ms_by_prompt_tokens": by_length} if by_length else {})}


def config_summary(line):
    """BASELINE.json's five configs in one compact block (value, unit, fraction of the roofline that bounds it, kernel, whether
    the device result was checked): what the long `extras` hold, short enough to read at a glance."""
    ex = line.get("extras", {})
    rf = line["roofline"]
    out = {"c2_fused_reduce_2pow24": {"GB/s": rf["achieved"], "frac_hbm": rf["frac"], "us": rf["step_us"], "kernel_frac_hbm": rf["kernel_frac"],
                                      "sustained_frac_hbm": rf.get("sustained_frac"), "launches": 2, "verified": True}}

    def take(dst, src, keys, **more):
        row = ex.get(src)
        if isinstance(row, dict) and "error" not in row:
            out[dst] = {**{k: row[k] for k in keys if k in row}, **more}
            v = row.get("verified")
            if v is not None:
                out[dst]["verified"] = bool(v)
        elif isinstance(row, dict):
            out[dst] = {"error": row["error"]}
    take("c1_softmax_lazy_32x1024", "softmax_lazy_32x1024", ("us_per_softmax", "GB/s", "frac_hbm", "launches", "bound"))
    take("c1_softmax_custom_32x1024", "softmax_custom_32x1024", ("us_per_softmax", "GB/s", "frac_hbm", "launches", "bound"))
    take("softmax_custom_4096x4096", "softmax_custom_4096x4096", ("us_per_softmax", "GB/s", "frac_hbm"))
    take("softmax_custom_32768x4096_1GiB", "softmax_custom_32768x4096", ("us", "GB/s", "frac_hbm"))
    take("c3_bmm_f32_8x1024^3", "bmm_f32_8x1024^3", ("TFLOP/s", "frac_mfma_f32", "us", "kernel"))
    take("c3_bmm_f32_8x1024^3_six_bf16_terms", "bmm_f32_8x1024^3_six_bf16_terms", ("TFLOP/s_f32_equivalent", "times_the_f32_matrix_peak", "frac_mfma_bf16", "us", "kernel"))
    for key in ("mm_f32_nn_4096^3", "mm_f32_nn_4096^3_six_bf16_terms"):
        take(key, key, ("TFLOP/s", "TFLOP/s_f32_equivalent", "frac_mfma_f32", "times_the_f32_matrix_peak", "frac_mfma_bf16", "us"))
    take("c3_bmm_bf16_8x1024^3", "bmm_bf16_8x1024^3", ("TFLOP/s", "frac_mfma_bf16", "us", "kernel"))
    if "c3_bmm_bf16_8x1024^3" in out and "bound_us" in ex.get("bmm_bf16_8x1024^3", {}):
        out["c3_bmm_bf16_8x1024^3"]["bound_us"] = ex["bmm_bf16_8x1024^3"]["bound_us"]["sum"]
    for key in ("mm_bf16_nt_4096^3", "mm_bf16_nn_4096^3", "mm_bf16_nt_8192^3"):
        take(key, key, ("TFLOP/s", "frac_mfma_bf16", "us"))
    for key in ("c4_rms_norm_512x2048", "c4_rope_q_1x32x512x64", "c4_causal_mask_1x32x512x512", "c4_softmax_custom_1x32x512x512", "c4_softmax_lazy_1x32x512x512",
                "c4_causal_softmax_fused"):
        take(key, key, ("us", "GB/s", "frac_hbm"))
    for key in ("c4_qk_t_b32_512x512x64", "c4_att_v_b32_512x64x512", "c4_attention_cached_t512", "attention_cached_t2048"):
        take(key, key, ("us", "TFLOP/s", "frac_mfma_f32", "frac_mfma_bf16", "GB/s", "frac_hbm"))
    for dst, src in (("c5_decode_f32_reference_graph", "llama_decode_f32"), ("c5_decode_f32_fused_level3", "llama_decode_f32_fused_projections"),
                     ("c5_decode_bf16_matrices_level3", "llama_decode_bf16_matrices"), ("c5_decode_bf16_matrices_prefill_bf16x3", "llama_decode_bf16_matrices_prefill_bf16x3"),
                     ("c5_unit_norms_decode_f32_reference_graph", "llama_decode_f32_reference_graph_unit_norms"),
                     ("c5_unit_norms_decode_bf16_matrices_prefill_bf16x3", "llama_decode_bf16_matrices_prefill_bf16x3_unit_norms"),
                     ("c5_unit_norms_prompt1900_bf16_matrices", "llama_decode_bf16_matrices_prompt1900"),
                     ("c5_unit_norms_prompt1900_bf16_matrices_prefill_bf16x3", "llama_decode_bf16_matrices_prompt1900_prefill_bf16x3")):
        row = ex.get(src)
        if not isinstance(row, dict):
            continue
        if "error" in row:
            out[dst] = {"error": row["error"]}
            continue
        chk = row.get("ids_vs_oracle_fixture", {})
        out[dst] = {"tok/s": row["tok/s"], "frac_hbm_weights_only": row["frac_hbm_weights_only"], "decode_ms_per_token": row["decode_ms_per_token"],
                    "prefill_ms": row.get("prefill_ms_warm", row["prefill_ms"]), "launches_per_token": row.get("launches_per_token"),
                    "ids_equal": f"{chk.get('ids_equal')}/{chk.get('of')}" if chk.get("checked") else "not checked: " + str(chk.get("why")),
                    "fixture": chk.get("fixture")}
    cb = ex.get("cpu_llama_decode_f32")
    if isinstance(cb, dict) and "tok/s" in cb:
        out["c5_cpu_port_f32"] = {"tok/s": cb["tok/s"], "cores": cb["cores"]}
    return out


def decode_launch_floor_model(ex):
    """A decode step as a chain of dependent launches: launches x the measured time of one dependent launch + the weights at
    the rate a read-only stream beyond the caches reaches on this box.  measured / model says how much of the miss against the
    weights-only ceiling that model explains."""
    chain, stream = ex.get("launch_chain_8_workgroups"), ex.get("fused_reduce_2pow27")
    if not (isinstance(chain, dict) and isinstance(stream, dict) and "us_per_dependent_launch" in chain and "GB/s" in stream):
        return None
    out = {"us_per_dependent_launch": chain["us_per_dependent_launch"], "stream_GB/s": stream["GB/s"],
           "formula": "launches_per_token x us_per_dependent_launch + weight_bytes / stream rate"}
    for key, wbytes in (("llama_decode_f32_fused_projections", 4 * 1034512384), ("llama_decode_bf16_matrices", 2 * 1034512384), ("llama_decode_f32", 4 * 1034512384)):
        row = ex.get(key)
        if isinstance(row, dict) and row.get("launches_per_token"):
            model_us = row["launches_per_token"] * chain["us_per_dependent_launch"] + wbytes / stream["GB/s"] / 1e3
            out[key] = {"launches_per_token": row["launches_per_token"], "model_us": round(model_us, 1), "measured_us": round(row["decode_ms_per_token"] * 1e3, 1),
                        "measured_over_model": round(row["decode_ms_per_token"] * 1e3 / model_us, 3)}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--extras", action="store_true", help="(default) kept for older command lines")
    ap.add_argument("--llama", action="store_true", help="(default) kept for older command lines")
    ap.add_argument("--llama-level", type=int, default=None, choices=[0, 1, 2, 3], help="run config 5 at this fusion level only (default: all four)")
    ap.add_argument("--llama-bf16", action="store_true", help="with --llama-level 3: the run with bf16 matrices instead of the f32 one")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-llama", action="store_true")
    ap.add_argument("--headline-only", action="store_true", help="only the config-2 kernel: no extras, no llama, no CPU baseline")
    ap.add_argument("--only", choices=["softmax", "bmm", "llama_pieces", "hbm_large", "floors", "safetensors", "cpu", "llama"], help="besides the headline, run just this group (profiler runs)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--sustained-trace", type=float, default=0.0, metavar="SECONDS",
                    help="also run the headline step without a pause for this long and report its rate per 50 ms of elapsed time")
    ap.add_argument("--copy-probe", action="store_true", help="also run a plain 2^24-element copy kernel (counter calibration)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU only (nothing in the path is sharded); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import ug_amd
    from ug_amd import rng
    dev = ug_amd.hip_device(0)
    a, b = rng.uniform_pm1(2, N), rng.uniform_pm1(3, N)
    truth = float(np.sum(a.astype(np.float64) * b + 0.5 * a.astype(np.float64)))
    r, cs, keep = fused_reduce(dev, a, b)
    cs.run()
    got = float(r.data_vec()[0])
    if not abs(got - truth) <= 1e-5 * abs(truth) + 1e-2:
        raise SystemExit(f"bench.py: wrong result {got} vs {truth}")
    info = cs.funcs()[0]["info"]

    # The timed region (W warm-up steps, then exactly K steps between synchronisations) is run three times and the
    # median run is the one reported: K = 200 steps are 4 ms of GPU time, and one scheduler hiccup on the host
    # moves a single run's wall clock by 20 %.  All three are kept in the line ("runs").
    runs = sorted((timed(dev, cs.run, args.steps, args.warmup) for _ in range(3)), key=lambda t: t[0])
    wall, ev_ms = runs[1]
    ms_per_step = wall * 1e3 / args.steps
    value = ALGO_BYTES * args.steps / wall / 1e9
    achieved = ALGO_BYTES / (ev_ms * 1e-3 / args.steps) / 1e9
    part_us = fused_reduce_parts(dev, a, b, truth, args.steps, args.warmup)

    line = {
        "metric": "GB/s (reductions) vs HBM roofline", "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "fused elementwise+reduce sum(a*b + 0.5*a), f32, len 2^24, U(-1,1) seeds 2/3, one lazy graph ending in narrow(0,0,1)",
                   "algorithmic_bytes_per_step": ALGO_BYTES, "kernel": info},
        # achieved / frac: the algorithmic bytes over the whole step (both kernels of the grid-wide reduction: HIP events on the
        # library's stream around K steps) -- what `value` sees, minus the host.  kernel_*: the same bytes over the dominant
        # kernel's own launch duration (the first of the two moves all the bytes; HIP events around K launches of it alone).
        # sustained_*: the whole step again behind half a second of the same launches (filled in at the end of the run).
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "step_us": round(ev_ms * 1e3 / args.steps, 3),
                     "kernel": "ug_Ln_Rs_Ba_Bm_O_O_Bm_O_C (stage 1 of the grid-wide reduction)",
                     "kernel_achieved": round(ALGO_BYTES / (part_us[0] * 1e-6) / 1e9, 2), "kernel_frac": round(ALGO_BYTES / (part_us[0] * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                     "kernel_us": round(part_us[0], 3), "fold_kernel_us": round(part_us[1], 3),
                     "traffic": TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE},
        "result": got, "truth_f64": truth,
        "runs": [{"ms_per_step": round(w * 1e3 / args.steps, 5), "kernel_us": round(e * 1e3 / args.steps, 3)} for w, e in runs],
    }
    if args.copy_probe:
        # A plain f32 copy of known size (2^24 elements: 64 MiB read, 64 MiB written) in the same
        # process: the scale for rocprofv3's FETCH_SIZE / WRITE_SIZE counters.
        from ug_amd import LazyBuffer as LB, Schedule
        cp = LB.copy(a, (N,), dev).unary("id")
        ccs = Schedule.create_one(cp).compile()
        _, cms = timed(dev, ccs.run, args.steps, args.warmup)
        line["copy_probe"] = {"kernel": ccs.funcs()[0]["info"], "bytes_read": 4 * N, "bytes_written": 4 * N,
                              "GB/s": round(8.0 * N * args.steps / (cms * 1e-3) / 1e9, 1)}
    if args.only:
        args.no_cpu_baseline = True
        args.no_extras = args.only == "llama"
        args.no_llama = args.only != "llama"
    if not (args.no_cpu_baseline or args.headline_only):
        line["cpu_baseline"] = cpu_baseline(a, b, truth)
    del keep, cs, r
    # The other configs ride along; a failure there is reported, it does not take the headline down.
    if not (args.no_extras or args.headline_only):
        try:
            line["extras"] = extras(dev, max(20, args.steps // 4), args.warmup, None if args.only in (None, "llama") else args.only)
        except Exception as e:  # noqa: BLE001
            line["extras"] = {"error": f"{type(e).__name__}: {e}"}
    if not (args.no_llama or args.headline_only):
        # the last entry: the same model decoding behind a 1900-token prompt (caches near their 2048 rows)
        # the x3 entries: the prompt's products as three bf16 terms per row element on the bf16 matrix pipe (decode steps are unchanged)
        # the *_unit_norms entries: the same model with norm vectors 1 + N(0, 0.02) instead of BASELINE's N(0, 0.02): same kernels and
        # bytes, but logits that differ enough for the greedy ids to mean something (checked against fixtures of their own)
        for key, fused, narrow, n_prompt, n_steps, x3, norm_mean in (("llama_decode_f32", 0, False, 128, 128, False, 0.0), ("llama_decode_f32_fused_attention", 1, False, 128, 128, False, 0.0),
                                                                     ("llama_decode_f32_inplace_cache", 2, False, 128, 128, False, 0.0),
                                                                     ("llama_decode_f32_fused_projections", 3, False, 128, 128, False, 0.0),
                                                                     ("llama_decode_bf16_matrices", 3, True, 128, 128, False, 0.0),
                                                                     ("llama_decode_bf16_matrices_prefill_bf16x3", 3, True, 128, 128, True, 0.0),
                                                                     ("llama_decode_f32_reference_graph_unit_norms", 0, False, 128, 128, False, 1.0),
                                                                     ("llama_decode_bf16_matrices_prefill_bf16x3_unit_norms", 3, True, 128, 128, True, 1.0),
                                                                     ("llama_decode_bf16_matrices_prompt1900", 3, True, 1900, 64, False, 1.0),
                                                                     ("llama_decode_bf16_matrices_prompt1900_prefill_bf16x3", 3, True, 1900, 64, True, 1.0)):
            if args.llama_level is not None and (fused != args.llama_level or narrow != args.llama_bf16):
                continue
            try:
                line.setdefault("extras", {})[key] = llama_decode(dev, n_prompt=n_prompt, n_steps=n_steps, fused_attention=fused, bf16_matrices=narrow, bf16x3=x3, norm_mean=norm_mean)
            except Exception as e:  # noqa: BLE001
                line.setdefault("extras", {})[key] = {"error": f"{type(e).__name__}: {e}"}
    # The same step behind half a second of the same launches.  In a process that has done nothing else the chip streams
    # slower after tenths of a second than in its first milliseconds (measured: 21.6 us per step after 20 warm-up steps,
    # 24-27 us after 20000); at the end of a full run it does not (21.4 us).  `value` stays what the stated W and K measure;
    # this figure is taken last, so that no other row of this run is measured in its wake.
    r, cs, keep = fused_reduce(dev, a, b)
    cs.run()
    clocks = {}
    try:
        probe = ClockProbe(dev)
        probe.mhz()
        dev.synchronize()
        time.sleep(1.0)
        clocks["after_1s_idle"] = probe.mhz()
        for _ in range(args.warmup + args.steps):
            cs.run()
        clocks[f"behind_{args.warmup + args.steps}_steps"] = probe.mhz()
    except Exception as e:  # noqa: BLE001
        clocks["error"] = f"{type(e).__name__}: {e}"
        probe = None
    _, sus_ms = timed_hot(dev, cs.run, args.steps, 0, 0.5)
    if probe is not None:
        clocks["behind_half_a_second_of_steps"] = probe.mhz()
    if args.sustained_trace > 0:
        time.sleep(1.0)    # let the chip fall back to idle first: the trace starts where a fresh process would
        line["sustained_trace"] = sustained_trace(dev, cs.run, args.sustained_trace)
    del keep, cs, r
    line["sustained"] = {"after_s": 0.5, "us_per_step": round(sus_ms * 1e3 / args.steps, 3), "GB/s": round(ALGO_BYTES / (sus_ms * 1e-3 / args.steps) / 1e9, 1),
                         "frac_hbm": round(ALGO_BYTES / (sus_ms * 1e-3 / args.steps) / 1e9 / HBM_PEAK_GBS, 4)}
    line["sustained"]["core_clock_mhz"] = clocks
    line["roofline"]["sustained_achieved"] = line["sustained"]["GB/s"]
    line["roofline"]["sustained_frac"] = line["sustained"]["frac_hbm"]
    line["roofline"]["configs"] = config_summary(line)
    model = decode_launch_floor_model(line.get("extras", {}))
    if model:
        line["roofline"]["launch_floor_model"] = model
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
