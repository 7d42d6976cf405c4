#!/usr/bin/env python3
"""Headline benchmark: GPT-2-small shaped, GGUF-Q8_0 weights, batch-1 greedy decode on one MI355X.

A "step" is one decode step (one token).  Weights, KV cache, token and position are resident in
HBM before the timed region; the timed region is K back-to-back steps of the device-resident loop
(cthip_decoder_generate), bracketed by stream synchronisation, host wall clock.  `roofline` is
the whole decode step (one hipGraph replay) measured with HIP events on the library's stream:
algorithmic bytes of a step (packed weights + norms/biases + embedding rows + KV rows) over its
average duration, against 8 TB/s.  `cpu_baseline` times the CPU oracle (a single-thread C
restatement of Caten's BACKEND=CLANG kernels, incl. its one-hot embedding and 3-reduction argmax)
on the host cores, on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def cpu_baseline(cfg, weights, prompt, budget_s):
    """Oracle ("port" of the CLANG path), one thread: decode steps at the same positions."""
    import oracle
    from caten_amd import synth
    from caten_amd.llm import Tensor
    wd = dict(weights)
    for k in synth.GPT2_LINEAR_KEYS:
        wd[k] = [oracle.dequant("q8_0", Tensor.from_f32(a, "q8_0").raw, a.size).reshape(a.shape) for a in weights[k]]
    wd["lm_head"] = oracle.dequant("q8_0", Tensor.from_f32(weights["lm_head"], "q8_0").raw,
                                   weights["lm_head"].size).reshape(weights["lm_head"].shape)
    m = oracle.GPT2(cfg, wd)
    # prefill untimed and with the row-copy embedding so the sample is decode steps only
    tok, _ = m.forward([float(t) for t in prompt], 0, onehot=False, all_logits=False)
    n = len(prompt)
    steps, t0 = 0, time.perf_counter()
    while True:
        tok, _ = m.forward([float(tok)], n, onehot=True, all_logits=True)
        n += 1
        steps += 1
        el = time.perf_counter() - t0
        if el >= budget_s or steps >= 64:
            break
    return {"value": steps / el, "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": f"{steps} decode steps after a {len(prompt)}-token prompt, fp32 dequantised weights, "
                      f"gcc -O3 single thread (what BACKEND=CLANG runs at OMP=0), {el:.1f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--model", default="gpt2")
    ap.add_argument("--kind", default="q8_0")
    ap.add_argument("--prompt", type=int, default=16)
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="CPU baseline budget (0 disables)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (batch-1 decode does not use a second); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import ctypes as C
    from caten_amd import _lib, synth, llm
    cfg = dict(synth.GPT2_CONFIGS[args.model])
    weights = synth.gpt2_weights(cfg, seed=0)
    prompt = synth.prompt(cfg["vocab"], args.prompt, seed=0)
    total = args.warmup + args.steps
    if args.prompt + total + 1 > cfg["max_seq"]:
        # the KV cache bounds how many tokens one sequence can hold: restart sequences as needed
        pass
    lib = _lib.init(0)
    model = llm.make_gpt2(cfg, llm.gpt2_state_dict(weights, args.kind))

    def run(n_steps):
        """n_steps decode steps, restarting from the prompt whenever the KV cache is full."""
        done = 0
        positions = []
        while done < n_steps:
            if model.position == 0 or model.position + 1 > cfg["max_seq"] - 1:
                model.forward([float(t) for t in prompt], len(prompt), 0)
            room = cfg["max_seq"] - model.position
            k = min(n_steps - done, room)
            positions.extend(range(model.position, model.position + k))
            model.generate_on_device(k)
            done += k
        return positions

    model.forward([float(t) for t in prompt], len(prompt), 0)  # prefill, untimed
    if args.warmup:
        run(args.warmup)
    if model.position + args.steps > cfg["max_seq"]:
        model.forward([float(t) for t in prompt], len(prompt), 0)
    _lib.check(lib.cthip_sync())

    # ---- timed region: exactly K decode steps ----
    t0 = time.perf_counter()
    positions = run(args.steps)
    _lib.check(lib.cthip_sync())
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    tok_s = args.steps / wall

    # ---- roofline of the step kernel sequence, HIP events on the launch stream ----
    if model.position + args.steps > cfg["max_seq"]:
        model.forward([float(t) for t in prompt], len(prompt), 0)
    k = min(args.steps, cfg["max_seq"] - model.position)
    pos0 = model.position
    out = np.empty(k, np.int64)
    _lib.check(lib.cthip_sync())
    _lib.check(lib.cthip_timer_start())
    _lib.check(lib.cthip_decoder_generate(model.handle, k, out.ctypes.data))
    ms = C.c_float()
    _lib.check(lib.cthip_timer_stop(C.byref(ms)))
    step_us = ms.value * 1e3 / k
    step_bytes = float(np.mean([model.step_bytes(t + 1) for t in range(pos0, pos0 + k)]))
    achieved = step_bytes / (step_us * 1e-6) / 1e9

    res = {
        "metric": "decode tokens/sec at batch 1 on 1 MI355X; fused-kernel HBM GB/s vs peak",
        "value": tok_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"GPT-2-small shape ({cfg['n_layers']}L d{cfg['dim']} h{cfg['n_heads']} ffn{cfg['ffn']} "
                               f"vocab{cfg['vocab']}), GGUF-{args.kind.upper()} linear weights, fp32 embeddings/LayerNorm/KV, "
                               f"{args.prompt}-token prompt, batch-1 greedy decode, positions {min(positions)}..{max(positions)}",
                   "model": args.model, "weights": args.kind, "batch": 1},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "kernel": "one decode step (hipGraph of the fused GEMV/attention/argmax launches)",
                     "bytes_per_step": step_bytes, "us_per_step": step_us},
    }
    if args.cpu_seconds > 0:
        res["cpu_baseline"] = cpu_baseline(cfg, weights, prompt, args.cpu_seconds)
    model.close()
    print(json.dumps(res))


if __name__ == "__main__":
    main()
