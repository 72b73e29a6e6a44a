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
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0           # MI355X HBM3E, vendor figure
MFMA_BF16_PEAK_TF = 2500.0      # dense bf16
MFMA_F32_PEAK_TF = 157.3        # f32 matrix
N = 1 << 24
ALGO_BYTES = 2 * N * 4 + 4      # read a, read b, write one f32

# HBM bytes per step from `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE`, scaled by the counters'
# reading for the --copy-probe kernel (profiles/fused_reduce_2pow24_hbm_traffic.txt).
TRAFFIC_BYTES = 134222039


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


def fused_reduce(dev, a, b):
    import ref_suite
    from ug_amd import LazyBuffer as LB, Schedule
    la, lb = LB.copy(a, (a.size,), dev), LB.copy(b, (b.size,), dev)
    r = ref_suite.fused_reduce_graph(la, lb, dev)
    cs = Schedule.create_one(r).compile()
    return r, cs, (la, lb)


def cpu_baseline(a, b, truth, budget_s=12.0):
    """The CPU oracle (restatement of ug's CPU backend: same emitted C, same gcc flags, one thread)
    on the same workload, timed on this box's host cores."""
    from conftest import _oracle_lib
    import ug_amd
    lib = _oracle_lib()
    out = C.c_void_p()
    assert lib.ugo_cpu_device_new(C.byref(out)) == 0
    cpu = ug_amd.Device(out.value)
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


def cpu_extras(budget_s=4.0):
    """The CPU oracle (restatement of ug's CPU backend) on configs 1 and 3, timed on this box's host
    cores next to the GPU numbers: each a bounded sample of the same workload."""
    from conftest import _oracle_lib
    import ug_amd
    from ug_amd import LazyBuffer as LB, Schedule, rng
    lib = _oracle_lib()
    h = C.c_void_p()
    assert lib.ugo_cpu_device_new(C.byref(h)) == 0
    cpu = ug_amd.Device(h.value)
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
    # config 5 at full width, two of the 22 layers: a decode step is the same two layers 11 times over
    # plus the head, so the per-layer and the head time are fitted from a 1-layer and a 2-layer run
    prompt = rng.token_ids(10, 8, 32000)
    oh = C.c_void_p()
    assert lib.ugo_llama_ops_cpu(C.byref(oh)) == 0
    cpu_ops = ug_amd.LlamaOps(oh.value)
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
    """Other single-GPU configs of BASELINE.json: GB/s or TFLOP/s with the roofline fraction."""
    out = {}
    if only in (None, "softmax"):
        out.update(softmax_sweep(dev, steps, warmup))
    if only in (None, "bmm"):
        out.update(bmm(dev, steps, warmup))
    if only in (None, "llama_pieces"):
        out.update(llama_pieces(dev, steps, warmup))
    if only in (None, "safetensors"):
        out.update(safetensors_load(dev))
    if only in (None, "cpu"):
        out.update(cpu_extras())
    return out


def safetensors_load(dev, n=1 << 27):
    """A 256 MiB bf16 tensor in a safetensors file (page cache warm) loaded as f32: upload + widen
    on the device against widen on the host + upload (the order of ug-core/src/safetensors.rs:141-271),
    and the widening kernel alone (6 bytes per element)."""
    import tempfile
    import st_files
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
        ops = ug_amd.LlamaOps.hip()
        cm = ops.custom_softmax(src)
        cs2 = Schedule.create_one(cm).compile()
        _, ms = timed(dev, cs2.run, steps, warmup)
        gbs = 8.0 * rows * cols * steps / (ms * 1e-3) / 1e9
        out[f"softmax_custom_{rows}x{cols}"] = {"GB/s": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4), "us_per_softmax": round(ms * 1e3 / steps, 2),
                                               "launches": 1}
    return out


def bmm(dev, steps, warmup):
    """Config 3: batched matmul 8 x 1024^3, f32 through the lazy graph and bf16 through Device::matmul."""
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
    _, ms = timed(dev, cs.run, steps, warmup)
    tf = flop * steps / (ms * 1e-3) / 1e12
    out["bmm_f32_8x1024^3"] = {"TFLOP/s": round(tf, 2), "frac_mfma_f32": round(tf / MFMA_F32_PEAK_TF, 4), "us": round(ms * 1e3 / steps, 1)}
    sa, sw = dev.slice_from(rng.to_bf16_bits(a)), dev.slice_from(rng.to_bf16_bits(w))
    dst = dev.allocate_uninit(ug_amd.BF16, b * m * m)
    lay = ((b, m, m), (m * m, m, 1), 0)
    _, ms = timed(dev, lambda: dev.matmul(dst, sa, sw, (b, m, m, m), lay, lay), steps, warmup)
    tf = flop * steps / (ms * 1e-3) / 1e12
    out["bmm_bf16_8x1024^3"] = {"TFLOP/s": round(tf, 2), "frac_mfma_bf16": round(tf / MFMA_BF16_PEAK_TF, 4), "us": round(ms * 1e3 / steps, 1)}
    # a large product with the rhs stored [n, k] (what matmul_t of the llama projections hands over): 256 tiles of 256 x 256
    m = 4096
    a, w = rng.uniform_pm1(4, m * m), rng.uniform_pm1(5, m * m)
    sa, sw = dev.slice_from(rng.to_bf16_bits(a)), dev.slice_from(rng.to_bf16_bits(w))
    dst = dev.allocate_uninit(ug_amd.BF16, m * m)
    _, ms = timed(dev, lambda: dev.matmul(dst, sa, sw, (1, m, m, m), ((1, m, m), (m * m, m, 1), 0), ((1, m, m), (m * m, 1, m), 0)), steps, warmup)
    tf = 2.0 * m * m * m * steps / (ms * 1e-3) / 1e12
    out["mm_bf16_nt_4096^3"] = {"TFLOP/s": round(tf, 2), "frac_mfma_bf16": round(tf / MFMA_BF16_PEAK_TF, 4), "us": round(ms * 1e3 / steps, 1)}
    return out


def llama_pieces(dev, steps, warmup):
    """Config 4: the llama layer pieces at T=512, hidden 2048, 32 heads x 64 (f32), each as the lazy
    graph ug-llama builds for it (ug-llama/src/model.rs:32-109,203-248), with its algorithmic bytes."""
    import ug_amd
    from ug_amd import LazyBuffer as LB, Schedule, rng
    ll, ops = ug_amd.llama, ug_amd.LlamaOps.hip()
    out = {}
    t, hidden, heads, hd = 512, 2048, 32, 64

    def hbm(name, lb, nbytes, keep=()):
        cs = Schedule.create_one(lb).compile()
        _, ms = timed(dev, cs.run, steps, warmup)
        gbs = nbytes * steps / (ms * 1e-3) / 1e9
        out[name] = {"GB/s": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4), "us": round(ms * 1e3 / steps, 2), "algorithmic_bytes": nbytes}

    x = LB.copy(rng.normal(6, t * hidden), (1, t, hidden), dev)
    alpha = LB.copy(rng.normal(6 + 100, hidden, 0.02), (hidden,), dev)
    hbm("c4_rms_norm_512x2048", ll.rms_norm(x, alpha, 1e-5), 2 * 4 * t * hidden + 4 * hidden)
    cfg = ug_amd.LlamaConfig()
    cos, sin = ll.rope_tables(dev, cfg)
    cos.realize()   # the tables are built once per model (ug-llama/src/model.rs:147-168), not per layer call
    sin.realize()
    q = LB.copy(rng.normal(7, heads * t * hd), (1, heads, t, hd), dev)
    pos = LB.copy(np.zeros(1, np.int32), (1,), dev)
    hbm("c4_rope_q_1x32x512x64", ops.rope(q, cos, sin, pos), 2 * 4 * heads * t * hd + 2 * 4 * t * (hd // 2))
    s = LB.copy(rng.normal(8, heads * t * t), (1, heads, t, t), dev)
    hbm("c4_causal_mask_1x32x512x512", ops.causal_mask(s), 2 * 4 * heads * t * t)
    hbm("c4_softmax_lazy_1x32x512x512", ll.softmax(s), 2 * 4 * heads * t * t)
    hbm("c4_softmax_custom_1x32x512x512", ops.custom_softmax(s), 2 * 4 * heads * t * t)
    hbm("c4_mask_then_softmax_custom", ops.custom_softmax(ops.causal_mask(s)), 4 * 4 * heads * t * t)
    # the same two ops as one kernel: reads the kept triangle, writes every element
    hbm("c4_causal_softmax_fused", ops.causal_softmax(s), 2 * 4 * heads * t * t)
    gate = LB.copy(rng.normal(8 + 100, t * 5632), (1, t, 5632), dev)
    up = LB.copy(rng.normal(8 + 101, t * 5632), (1, t, 5632), dev)
    hbm("c4_silu_mul_512x5632", ll.silu(gate).binary("mul", up), 3 * 4 * t * 5632)

    def gemm(name, lhs, rhs, transposed, b, m, n, k):
        mm = lhs.matmul_t(rhs) if transposed else lhs.matmul(rhs)
        cs = Schedule.create_one(mm).compile()
        _, ms = timed(dev, cs.run, steps, warmup)
        flop, nbytes = 2.0 * b * m * n * k, 4.0 * b * (m * k + k * n + m * n)
        sec = ms * 1e-3 / steps
        out[name] = {"TFLOP/s": round(flop / sec / 1e12, 2), "frac_mfma_f32": round(flop / sec / 1e12 / MFMA_F32_PEAK_TF, 4), "GB/s": round(nbytes / sec / 1e9, 1),
                     "frac_hbm": round(nbytes / sec / 1e9 / HBM_PEAK_GBS, 4), "us": round(sec * 1e6, 2)}

    kk = LB.copy(rng.normal(8 + 200, heads * t * hd), (1, heads, t, hd), dev)
    v = LB.copy(rng.normal(8 + 300, heads * t * hd), (1, heads, t, hd), dev)
    gemm("c4_qk_t_b32_512x512x64", q, kk, True, heads, t, t, hd)
    gemm("c4_att_v_b32_512x64x512", s, v, False, heads, t, hd, t)

    # the whole chain either side of the softmax (rope(q), repeat, q k^T, scale, mask, softmax, x v, transposes) as one
    # kernel over preallocated caches of 4 kv heads: scores stay in registers.  flop = the two causal products.
    nkv, cap = 4, 2048
    qf = LB.copy(rng.normal(7, t * heads * hd), (1, t, heads * hd), dev)
    kc = LB.copy(rng.normal(8 + 200, nkv * cap * hd), (1, nkv, cap, hd), dev)
    vc = LB.copy(rng.normal(8 + 300, nkv * cap * hd), (1, nkv, cap, hd), dev)
    att = ops.attention_cached(qf, kc, vc, t, float(np.float32(hd) ** np.float32(-0.5)), cos, sin, pos, False)
    cs = Schedule.create_one(att).compile()
    _, ms = timed(dev, cs.run, steps, warmup)
    sec = ms * 1e-3 / steps
    flop = 2 * 2.0 * heads * hd * t * (t + 1) / 2
    nbytes = 4.0 * (2 * t * heads * hd + 2 * nkv * t * hd)
    out["c4_attention_cached_t512"] = {"us": round(sec * 1e6, 2), "TFLOP/s": round(flop / sec / 1e12, 2), "frac_mfma_f32": round(flop / sec / 1e12 / MFMA_F32_PEAK_TF, 4),
                                       "algorithmic_bytes": int(nbytes), "replaces": "c4_rope_q + c4_qk_t + c4_causal_softmax_fused + c4_att_v + 2 repeats + 2 transposes"}
    return out


def llama_decode(dev, n_prompt=128, n_steps=128, fused_attention=0, bf16_matrices=False):
    """Config 5: TinyLlama-1.1B shape, random-init f32 weights, prefill 128 then 128 greedy steps.
    Fresh buffers are not zero-filled here (every kernel of the model writes its whole output; the
    ids are the same either way, which the GPU tests check).  fused_attention: 0 = the reference's
    op-by-op graph; 1 = ughip_causal_softmax_rows / ughip_rope_append / ughip_attention_decode;
    2 = caches written in place (ughip_kv_append) and ughip_attention_cached for prefill and decode;
    3 = 2 plus packed q|k|v, gate/up + SwiGLU and residual projections (ughip_gemv_multi / _gate_up / _add).
    bf16_matrices: bf16-rounded weights, the projection matrices and the head kept and streamed as bf16
    (activations, caches, norms f32): the numbers of the f32 model on the rounded weights from half the bytes."""
    import ug_amd
    from ug_amd import rng
    cfg = ug_amd.LlamaConfig()
    ops = ug_amd.LlamaOps.hip()
    dev.set_zero_fill(False)
    t0 = time.perf_counter()
    model = ug_amd.LlamaModel(dev, ops, cfg, custom_softmax=True, seed=9, std=0.02, round_bf16=bf16_matrices, fused_attention=fused_attention,
                              bf16_matrices=bf16_matrices)
    load_s = time.perf_counter() - t0
    prompt = rng.token_ids(10, n_prompt, cfg.vocab_size)
    model.generate(prompt, 4)          # compiles every kernel shape family once
    toks, st = model.generate(prompt, n_steps)
    dev.set_zero_fill(True)
    # streamed per token: every matrix once (2 or 4 bytes per weight); the 45 norm vectors stay f32
    weights_bytes = (2 if bf16_matrices else 4) * 1034512384
    tok_s = n_steps / (st["decode_ms"] * 1e-3)
    return {"tok/s": round(tok_s, 2), "decode_ms_per_token": round(st["decode_ms"] / n_steps, 3), "prefill_ms": round(st["prefill_ms"], 1),
            "frac_hbm_weights_only": round(tok_s * weights_bytes / 1e9 / HBM_PEAK_GBS, 4), "load_s": round(load_s, 1), "dtype": "f32 activations, bf16 matrices" if bf16_matrices else "f32", "zero_fill": False, "fused_attention": fused_attention,
            "prompt_tokens": n_prompt, "decode_steps": n_steps, "first_ids": toks[:8].tolist(), "min_top1_margin": float(st["margins"].min())}


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
    ap.add_argument("--only", choices=["softmax", "bmm", "llama_pieces", "safetensors", "cpu", "llama"], help="besides the headline, run just this group (profiler runs)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
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

    line = {
        "metric": "GB/s (reductions) vs HBM roofline", "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "fused elementwise+reduce sum(a*b + 0.5*a), f32, len 2^24, U(-1,1) seeds 2/3, one lazy graph ending in narrow(0,0,1)",
                   "algorithmic_bytes_per_step": ALGO_BYTES, "kernel": info},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": TRAFFIC_BYTES, "kernel_us": round(ev_ms * 1e3 / args.steps, 3)},
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
        for key, fused, narrow, n_prompt, n_steps in (("llama_decode_f32", 0, False, 128, 128), ("llama_decode_f32_fused_attention", 1, False, 128, 128),
                                                      ("llama_decode_f32_inplace_cache", 2, False, 128, 128),
                                                      ("llama_decode_f32_fused_projections", 3, False, 128, 128),
                                                      ("llama_decode_bf16_matrices", 3, True, 128, 128),
                                                      ("llama_decode_bf16_matrices_prompt1900", 3, True, 1900, 64)):
            if args.llama_level is not None and (fused != args.llama_level or narrow != args.llama_bf16):
                continue
            try:
                line.setdefault("extras", {})[key] = llama_decode(dev, n_prompt=n_prompt, n_steps=n_steps, fused_attention=fused, bf16_matrices=narrow)
            except Exception as e:  # noqa: BLE001
                line.setdefault("extras", {})[key] = {"error": f"{type(e).__name__}: {e}"}
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
