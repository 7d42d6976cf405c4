#!/usr/bin/env python3
"""Headline benchmark: GPT-2-small shaped, GGUF-Q8_0 weights, batch-1 greedy decode on one MI355X.

A "step" is one decode step (one token).  Weights, KV cache, token and position are resident in
HBM before the timed region; the timed region is K back-to-back steps of the device-resident loop
(cthip_decoder_generate), bracketed by stream synchronisation, host wall clock.  `roofline` is the
whole step: algorithmic bytes of one token (packed weights + norms/biases + embedding rows + KV rows)
over the step time measured with HIP events on the library's stream, against 8 TB/s; its `lm_head`
entry gives the step's largest launch (50257x768, 31 % of the bytes) alone, once back to back on one
matrix (which then sits in the Infinity Cache) and once rotating over enough copies that every launch
streams from HBM.  `cpu_baseline` times the CPU oracle (a single-thread C restatement of Caten's
BACKEND=CLANG kernels, incl. its one-hot embedding and 3-reduction argmax) on the host cores, on a
bounded sample of the same workload.
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


def profile_traffic(model, kind):
    """HBM-side bytes of one decode step (FETCH_SIZE + WRITE_SIZE summed over the step's dispatches, scaled by a copy
    of known size) as recorded in the committed rocprofv3 --pmc summary of this workload; None if there is none."""
    path = os.path.join(ROOT, "profiles", f"decode_{model}_{kind}_step_pmc.txt")
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("step_traffic_bytes:"):
                    return int(float(line.split(":", 1)[1].split()[0]))
    except OSError:
        pass
    return None


def cpu_baseline(cfg, weights, prompt, budget_s, kind, llama):
    """Oracle ("port" of the CLANG path), one thread: decode steps at the same positions, on the
    dequantised fp32 weights (the reference has no quantised compute, dequantize.lisp:3-5)."""
    import oracle
    from caten_amd import synth
    from caten_amd.llm import Tensor
    wd = dict(weights)
    if kind != "f32":
        for k in (synth.LLAMA_LINEAR_KEYS if llama else synth.GPT2_LINEAR_KEYS):
            wd[k] = [oracle.dequant(kind, Tensor.from_f32(a, kind).raw, a.size).reshape(a.shape) for a in weights[k]]
        wd["lm_head"] = oracle.dequant(kind, Tensor.from_f32(weights["lm_head"], kind).raw,
                                       weights["lm_head"].size).reshape(weights["lm_head"].shape)
    m = oracle.Llama(cfg, wd) if llama else oracle.GPT2(cfg, wd)
    # prefill untimed (and with the row-copy embedding) so the sample is decode steps only
    tok, _ = m.forward([float(t) for t in prompt], 0) if llama else \
        m.forward([float(t) for t in prompt], 0, onehot=False, all_logits=False)
    n = len(prompt)
    steps, t0 = 0, time.perf_counter()
    while True:
        tok, _ = m.forward([float(tok)], n) if llama else m.forward([float(tok)], n, onehot=True, all_logits=True)
        n += 1
        steps += 1
        el = time.perf_counter() - t0
        if el >= budget_s or steps >= 64:
            break
    return {"value": steps / el, "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": f"{steps} decode steps after a {len(prompt)}-token prompt, fp32 dequantised weights, "
                      f"gcc -O3 single thread (what BACKEND=CLANG runs at OMP=0), {el:.1f} s",
            "items": cpu_baseline_items()}


def cpu_baseline_items():
    """The same port on bounded samples of the two single-item configurations that bench_items.py times on the GPU:
    relu(matmul) at 1024^3 (256 of the 1024 output rows) and the row ops of (64,1024,768) (half of the 65536 rows)."""
    import oracle
    rng = np.random.default_rng(0)
    out = {}
    A = rng.uniform(-1, 1, (256, 1024)).astype(np.float32)
    B = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    t0 = time.perf_counter()
    oracle.matmul(A, B, relu=True)
    el = time.perf_counter() - t0
    out["relu(matmul) 1024^3"] = {"value": 2.0 * 256 * 1024 * 1024 / el / 1e9, "unit": "GFLOP/s", "sample": f"256 of 1024 output rows, {el:.2f} s"}
    rows, d = 32768, 768
    x = rng.standard_normal((rows, d), dtype=np.float32)
    g, b = rng.normal(1, 0.02, d).astype(np.float32), rng.normal(0, 0.02, d).astype(np.float32)
    t0 = time.perf_counter()
    oracle.softmax(oracle.layernorm(x, g, b, 1e-5))
    el = time.perf_counter() - t0
    out["LayerNorm->softmax (64,1024,768)"] = {"value": 2.0 * rows * d * 4 / el / 1e9, "unit": "GB/s of the fused item's bytes",
                                               "sample": f"{rows} of 65536 rows, two kernels as the reference runs them, {el:.2f} s"}
    t0 = time.perf_counter()
    oracle.gelu_tanh(x)
    el = time.perf_counter() - t0
    out["GELU(tanh) (64,1024,768)"] = {"value": 2.0 * rows * d * 4 / el / 1e9, "unit": "GB/s", "sample": f"{rows} of 65536 rows, {el:.2f} s"}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--model", default="gpt2")
    ap.add_argument("--kind", default="q8_0")
    ap.add_argument("--prompt", type=int, default=16)
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="CPU baseline budget (0 disables)")
    ap.add_argument("--no-graph", action="store_true",
                    help="launch the step's kernels one by one instead of replaying the hipGraph (for kernel tracing)")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="library option set before the model is built (cthip_set_option), e.g. decode_fused=0")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (a kernel of known traffic to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings by)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (batch-1 decode does not use a second); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import ctypes as C
    from caten_amd import _lib, synth, llm
    llama = args.model in synth.LLAMA_CONFIGS
    cfg = dict(synth.LLAMA_CONFIGS[args.model] if llama else synth.GPT2_CONFIGS[args.model])
    weights = synth.llama_weights(cfg, seed=0) if llama else synth.gpt2_weights(cfg, seed=0)
    prompt = synth.prompt(cfg["vocab"], args.prompt, seed=0)
    total = args.warmup + args.steps
    if args.prompt + total + 1 > cfg["max_seq"]:
        # the KV cache bounds how many tokens one sequence can hold: restart sequences as needed
        pass
    lib = _lib.init(0)
    if args.no_graph:
        _lib.check(lib.cthip_set_option(b"decoder_graph", 0))
    for kv in args.option:
        name, value = kv.split("=")
        _lib.check(lib.cthip_set_option(name.encode(), int(value)))
    model = (llm.make_llama(cfg, llm.llama_state_dict(weights, args.kind)) if llama
             else llm.make_gpt2(cfg, llm.gpt2_state_dict(weights, args.kind)))

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
    # the same positions as the timed region above: restart from the prompt and redo the warm-up steps
    model.forward([float(t) for t in prompt], len(prompt), 0)
    if args.warmup:
        model.generate_on_device(min(args.warmup, cfg["max_seq"] - model.position - 1))
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
    step_gbs = step_bytes / (step_us * 1e-6) / 1e9

    # ---- the largest single launch of a step: ln_f -> lm_head GEMV (+ per-wavefront argmax partials) ----
    # "warm": the same matrix back to back -- 41 MB stay in the 256 MB Infinity Cache, so this is a cache-fed figure;
    # "cold": the launches rotate over enough copies of the matrix (> 256 MB together) that every one streams from HBM.
    from caten_amd import ops
    from caten_amd.llm import Tensor
    V, D = cfg["vocab"], cfg["dim"]
    t = Tensor.from_f32(weights["lm_head"], args.kind)
    wm0 = ops.WeightMatrix(args.kind, t.raw, V, D)
    ncopies = max(2, int(np.ceil(1.25 * (256 << 20) / wm0.nbytes)))
    wms = [wm0] + [ops.WeightMatrix(args.kind, t.raw, V, D) for _ in range(ncopies - 1)]
    dx = ops.DeviceArray.from_numpy(np.random.default_rng(1).normal(size=D).astype(np.float32))
    dg = ops.DeviceArray.from_numpy(weights["norm_w" if llama else "lnf_g"])
    db = None if llama else ops.DeviceArray.from_numpy(weights["lnf_b"])
    pro = _lib.PRO_RMSNORM if llama else _lib.PRO_LAYERNORM  # the final norm of the model, fused as the decode step fuses it
    dy = ops.DeviceArray((V,), np.float32)
    gemv_bytes = wm0.nbytes + 4 * ((2 if llama else 3) * D + V)  # packed weights + x, gamma (, beta) + logits

    def time_lm_head(mats, reps):
        for i in range(2 * len(mats)):
            _lib.check(lib.cthip_linear(dy.ptr, mats[i % len(mats)].handle, dx.ptr, 1, None, None, 0, pro, dg.ptr,
                                        db.ptr if db else None, 1e-5))
        _lib.check(lib.cthip_sync())
        _lib.check(lib.cthip_timer_start())
        for i in range(reps):
            _lib.check(lib.cthip_linear(dy.ptr, mats[i % len(mats)].handle, dx.ptr, 1, None, None, 0, pro, dg.ptr,
                                        db.ptr if db else None, 1e-5))
        _lib.check(lib.cthip_timer_stop(C.byref(ms)))
        us = ms.value * 1e3 / reps
        gbs = gemv_bytes / (us * 1e-6) / 1e9
        return {"us_per_launch": us, "achieved": gbs, "frac": gbs / HBM_PEAK_GBS}
    lm_warm = time_lm_head(wms[:1], 200)
    lm_cold = time_lm_head(wms, 25 * len(wms))
    lm_cold["copies"] = len(wms)
    # the streaming rate this box reaches: a 256 MiB device-to-device copy (read + written: twice that through HBM)
    ncopy = 256 << 20
    ca, cb = ops.DeviceArray((ncopy,), np.uint8), ops.DeviceArray((ncopy,), np.uint8)
    for _ in range(2):
        _lib.check(lib.cthip_d2d(cb.ptr, ca.ptr, ncopy))
    _lib.check(lib.cthip_sync())
    _lib.check(lib.cthip_timer_start())
    for _ in range(10):
        _lib.check(lib.cthip_d2d(cb.ptr, ca.ptr, ncopy))
    _lib.check(lib.cthip_timer_stop(C.byref(ms)))
    copy_gbs = 2.0 * ncopy / (ms.value * 1e-3 / 10) / 1e9
    lm_cold["frac_of_copy"] = lm_cold["achieved"] / copy_gbs
    ca.free()
    cb.free()
    traffic = profile_traffic(args.model, args.kind)

    res = {
        "metric": "decode tokens/sec at batch 1 on 1 MI355X; fused-kernel HBM GB/s vs peak",
        "value": tok_s, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{'Llama' if llama else 'GPT-2'} shape {args.model} ({cfg['n_layers']}L d{cfg['dim']} "
                               f"h{cfg['n_heads']} ffn{cfg['ffn']} "
                               f"vocab{cfg['vocab']}), GGUF-{args.kind.upper()} linear weights, fp32 embeddings/norms/KV, "
                               f"{args.prompt}-token prompt, batch-1 greedy decode, positions {min(positions)}..{max(positions)}",
                   "shape": args.model, "weight_format": args.kind, "prompt_tokens": args.prompt,
                   "positions": f"{min(positions)}..{max(positions)}"},
        # the whole decode step: every launch of one token, HIP events on the library's stream around K steps
        "roofline": {"bound": "hbm", "achieved": step_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": step_gbs / HBM_PEAK_GBS, "traffic": traffic,
                     "measured_copy": {"achieved": copy_gbs, "unit": "GB/s", "frac": copy_gbs / HBM_PEAK_GBS,
                                       "what": "256 MiB device-to-device copy on the library's stream, bytes read + written"},
                     "kernel": "one decode step = one replay of the step's launches (the dequant-in-register Linear "
                               "kernels, attention, argmax), packed weights + norms / biases + embedding rows + KV rows",
                     "bytes_per_launch": step_bytes, "us_per_launch": step_us,
                     "lm_head": {"kernel": f"cthip::k_gemv<{args.kind}> on lm_head ({V}x{D}) with the "
                                           f"{'RMSNorm' if llama else 'ln_f'} prologue, the step's largest launch",
                                 "bytes_per_launch": gemv_bytes, "warm_infinity_cache": lm_warm, "cold_hbm": lm_cold}},
    }
    if args.calibrate_copy:
        n = 256 << 20
        a, b = ops.DeviceArray((n,), np.uint8), ops.DeviceArray((n,), np.uint8)
        _lib.check(lib.cthip_d2d(b.ptr, a.ptr, n))
        _lib.check(lib.cthip_sync())
    if args.cpu_seconds > 0:
        res["cpu_baseline"] = cpu_baseline(cfg, weights, prompt, args.cpu_seconds, args.kind, llama)
    model.close()
    print(json.dumps(res))


if __name__ == "__main__":
    main()
