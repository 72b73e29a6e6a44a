#!/usr/bin/env python3
"""Writes tests/golden/llama_config5_greedy.json: what the CPU oracle (oracle/, the restatement of ug's CPU backend
running the op-by-op graph of ug-llama/src/model.rs) computes for BASELINE config 5 at its stated size --
22 layers, hidden 2048, 32/4 heads, FFN 5632, vocabulary 32000, N(0, 0.02) weights from seed 9, a prompt of 128
ids from seed 10, then 128 greedy steps -- once with f32 weights and once with the weights rounded to bf16.

    python tests/golden/make_llama_config5_fixture.py [--layers 22] [--prompt 128] [--steps 128]

Two more fixtures come from the same script.  BASELINE's weights make every norm vector N(0, 0.02): activations shrink
fifty-fold at each norm, the logits end up within 1e-4 of each other and the greedy ids fall into a two-cycle, so
equal ids say little there.  With the norm vectors at 1 + N(0, 0.02) -- what checkpoints hold -- logits spread
over several units and the ids carry information:

    python tests/golden/make_llama_config5_fixture.py --norm-mean 1 --out tests/golden/llama_config5_unit_norms_greedy.json
    python tests/golden/make_llama_config5_fixture.py --norm-mean 1 --prompt 1900 --steps 64 --out tests/golden/llama_config5_unit_norms_prompt1900_greedy.json

Per step it keeps the id picked, the largest logit and its gap to the second largest: the GPU tests hold the
HIP device to these position by position.  About ten minutes on 8 host cores; nothing here needs a GPU.
The values come from gcc-compiled kernels (-O3 -march=native -ffast-math): another host may differ in the
last bits, which is why the tests compare with a stated tolerance and treat near-ties by their margin.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=22)
    ap.add_argument("--prompt", type=int, default=128)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--norm-mean", type=float, default=0.0, help="norm vectors are this + N(0, 0.02)")
    ap.add_argument("--embed-std", type=float, default=0.0, help="embedding table (tied head) N(0, this) instead of N(0, 0.02)")
    ap.add_argument("--runs", default="f32,bf16_rounded")
    ap.add_argument("--out", default=os.path.join(ROOT, "tests", "golden", "llama_config5_greedy.json"))
    args = ap.parse_args()

    import ug_amd
    from ug_amd import rng
    from conftest import _oracle_lib
    lib = _oracle_lib()
    h, oh = C.c_void_p(), C.c_void_p()
    assert lib.ugo_cpu_device_new(C.byref(h)) == 0
    assert lib.ugo_llama_ops_cpu(C.byref(oh)) == 0
    cpu, cpu_ops = ug_amd.Device(h.value), ug_amd.LlamaOps(oh.value)
    os.environ.setdefault("RAYON_NUM_THREADS", str(os.cpu_count() or 1))

    cfg = ug_amd.LlamaConfig(num_hidden_layers=args.layers)
    prompt = rng.token_ids(10, args.prompt, cfg.vocab_size)
    out = {"config": {"num_hidden_layers": args.layers, "hidden_size": 2048, "intermediate_size": 5632, "num_attention_heads": 32,
                      "num_key_value_heads": 4, "vocab_size": 32000, "max_position_embeddings": 2048, "rope_theta": 10000.0, "rms_norm_eps": 1e-5},
           "weights": {"seed": 9, "std": 0.02, "norm_mean": args.norm_mean, "embed_std": args.embed_std}, "prompt": {"seed": 10, "n": args.prompt}, "steps": args.steps,
           "made_by": "tests/golden/make_llama_config5_fixture.py (CPU oracle, custom softmax, op-by-op graph)", "runs": {}}
    for key, round_bf16 in (("f32", False), ("bf16_rounded", True)):
        if key not in args.runs.split(","):
            continue
        t0 = time.perf_counter()
        model = ug_amd.LlamaModel(cpu, cpu_ops, cfg, custom_softmax=True, seed=9, std=0.02, round_bf16=round_bf16, norm_mean=args.norm_mean, embed_std=args.embed_std)
        toks, st = model.generate(prompt, args.steps)
        print(key, "done in", round(time.perf_counter() - t0, 1), "s; ids", toks[:8].tolist(), "min margin", float(st["margins"].min()), flush=True)
        out["runs"][key] = {"ids": toks.tolist(), "top1": [float(v) for v in st["top1"]], "margin": [float(v) for v in st["margins"]]}
        del model
    with open(args.out, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", args.out)


if __name__ == "__main__":
    main()
