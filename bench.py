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

The same JSON line carries, under `configs`, the other benchmark configurations measured in the same
run, each with its result checked before its figure is reported and each with its CPU-port sample:
relu(matmul) at 1024^3 (MFMA), the row ops of (64,1024,768) (HBM), the fp32 GPT-2-small decode, the
512-token prefill of the Q8_0 model (MFMA), the Llama-1.1B-shaped Q4_0 decode; and, under `byoc_path`,
the decode rate a Caten graph gets through the plug-in boundary: the compiled graph's node list walked
by the VM, one cthip_program_launch per Schedule-Item, the token back on the host after every forward
(apps/gpt2/gpt2.lisp:97-113).  `--configs headline` runs the headline workload only.
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
THREADS = min(16, os.cpu_count() or 1)


def profile_traffic(model, kind):
    """HBM-side bytes of one decode step (FETCH_SIZE + WRITE_SIZE summed over the step's dispatches, scaled by a copy
    of known size) and the positions they were counted at, as recorded in the committed rocprofv3 --pmc summary of
    this workload; (None, None) if there is none."""
    path = os.path.join(ROOT, "profiles", f"decode_{model}_{kind}_step_pmc.txt")
    traffic = positions = None
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("step_traffic_bytes:"):
                    traffic = int(float(line.split(":", 1)[1].split()[0]))
                if line.startswith("step_traffic_positions:"):
                    positions = line.split(":", 1)[1].strip()
    except OSError:
        pass
    return traffic, positions


def dequantised(weights, kind, llama):
    """the fp32 values the packed weights stand for (the reference has no quantised compute, dequantize.lisp:3-5)"""
    import oracle
    from caten_amd import synth
    from caten_amd.llm import Tensor
    if kind == "f32":
        return weights
    from concurrent.futures import ThreadPoolExecutor
    wd = dict(weights)

    def dq(a):
        return oracle.dequant(kind, Tensor.from_f32(a, kind).raw, a.size).reshape(a.shape)
    with ThreadPoolExecutor(THREADS) as pool:
        for k in (synth.LLAMA_LINEAR_KEYS if llama else synth.GPT2_LINEAR_KEYS):
            wd[k] = list(pool.map(dq, weights[k]))
        wd["lm_head"] = dq(weights["lm_head"])
    return wd


def cpu_decode(cfg, wd, prompt, budget_s, llama, max_steps=64):
    """Oracle ("port" of the CLANG path), one thread: decode steps after `prompt`.  Returns (tokens/s, tokens, text)."""
    import oracle
    m = oracle.Llama(cfg, wd) if llama else oracle.GPT2(cfg, wd)
    # prefill untimed (and with the row-copy embedding) so the sample is decode steps only
    tok, _ = m.forward([float(t) for t in prompt], 0) if llama else \
        m.forward([float(t) for t in prompt], 0, onehot=False, all_logits=False)
    toks = [tok]
    n = len(prompt)
    steps, t0 = 0, time.perf_counter()
    while True:
        tok, _ = m.forward([float(tok)], n) if llama else m.forward([float(tok)], n, onehot=True, all_logits=True)
        toks.append(tok)
        n += 1
        steps += 1
        el = time.perf_counter() - t0
        if el >= budget_s or steps >= max_steps:
            break
    return steps / el, toks, (f"{steps} decode steps after a {len(prompt)}-token prompt, fp32 dequantised weights, "
                              f"gcc -O3 single thread (what BACKEND=CLANG runs at OMP=0), {el:.1f} s")


def cpu_items():
    """The same port on bounded samples of the two single-item configurations:
    relu(matmul) at 1024^3 (256 of the 1024 output rows) and the row ops of (64,1024,768) (half of the 65536 rows)."""
    import oracle
    rng = np.random.default_rng(0)
    out = {}
    A = rng.uniform(-1, 1, (256, 1024)).astype(np.float32)
    B = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    t0 = time.perf_counter()
    oracle.matmul(A, B, relu=True)
    el = time.perf_counter() - t0
    out["relu(matmul) 1024^3"] = {"value": 2.0 * 256 * 1024 * 1024 / el / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": "port",
                                  "sample": f"256 of 1024 output rows, {el:.2f} s"}
    rows, d = 32768, 768
    x = rng.standard_normal((rows, d), dtype=np.float32)
    g, b = rng.normal(1, 0.02, d).astype(np.float32), rng.normal(0, 0.02, d).astype(np.float32)
    t0 = time.perf_counter()
    oracle.softmax(oracle.layernorm(x, g, b, 1e-5))
    el = time.perf_counter() - t0
    out["LayerNorm->softmax (64,1024,768)"] = {"value": 2.0 * rows * d * 4 / el / 1e9, "unit": "GB/s of the fused item's bytes", "cores": 1,
                                               "kind": "port", "sample": f"{rows} of 65536 rows, two kernels as the reference runs them, {el:.2f} s"}
    t0 = time.perf_counter()
    oracle.gelu_tanh(x)
    el = time.perf_counter() - t0
    out["GELU(tanh) (64,1024,768)"] = {"value": 2.0 * rows * d * 4 / el / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                                       "sample": f"{rows} of 65536 rows, {el:.2f} s"}
    return out


class Decode:
    """one decoder session and the measurements taken on it"""

    def __init__(self, lib, model_name, kind, weights, prompt):
        from caten_amd import synth, llm
        self.lib, self.kind, self.prompt = lib, kind, prompt
        self.llama = model_name in synth.LLAMA_CONFIGS
        self.cfg = dict(synth.LLAMA_CONFIGS[model_name] if self.llama else synth.GPT2_CONFIGS[model_name])
        self.model = (llm.make_llama(self.cfg, llm.llama_state_dict(weights, kind, threads=THREADS)) if self.llama
                      else llm.make_gpt2(self.cfg, llm.gpt2_state_dict(weights, kind)))

    def prefill(self):
        return self.model.forward([float(t) for t in self.prompt], len(self.prompt), 0)

    def run(self, n_steps):
        """n_steps decode steps, restarting from the prompt whenever the KV cache is full."""
        model, cfg = self.model, self.cfg
        done, positions = 0, []
        while done < n_steps:
            if model.position == 0 or model.position + 1 > cfg["max_seq"] - 1:
                self.prefill()
            k = min(n_steps - done, cfg["max_seq"] - model.position)
            positions.extend(range(model.position, model.position + k))
            model.generate_on_device(k)
            done += k
        return positions

    def timed(self, steps, warmup):
        """(wall seconds of exactly `steps` steps, their positions)"""
        from caten_amd import _lib
        self.prefill()
        if warmup:
            self.run(warmup)
        if self.model.position + steps > self.cfg["max_seq"]:
            self.prefill()
        _lib.check(self.lib.cthip_sync())
        t0 = time.perf_counter()
        positions = self.run(steps)
        _lib.check(self.lib.cthip_sync())
        return time.perf_counter() - t0, positions

    def events(self, steps, warmup):
        """the same positions again under HIP events on the library's stream: (us per step, mean algorithmic bytes)"""
        import ctypes as C
        from caten_amd import _lib
        model, cfg, lib = self.model, self.cfg, self.lib
        self.prefill()
        if warmup:
            model.generate_on_device(min(warmup, cfg["max_seq"] - model.position - 1))
        k = min(steps, cfg["max_seq"] - model.position)
        pos0 = model.position
        out = np.empty(k, np.int64)
        _lib.check(lib.cthip_sync())
        _lib.check(lib.cthip_timer_start())
        _lib.check(lib.cthip_decoder_generate(model.handle, k, out.ctypes.data))
        ms = C.c_float()
        _lib.check(lib.cthip_timer_stop(C.byref(ms)))
        step_bytes = float(np.mean([model.step_bytes(t + 1) for t in range(pos0, pos0 + k)]))
        return ms.value * 1e3 / k, step_bytes

    def first_tokens(self, n):
        """the prompt's token and the n - 1 greedy tokens after it (what the CPU port's tokens are compared with)"""
        tok = self.prefill()
        return [tok] + self.model.generate_on_device(n - 1)

    def close(self):
        self.model.close()


def decode_config(lib, name, model_name, kind, weights, prompt, steps, warmup, cpu_seconds, cpu_prompt=None, cpu_steps=64):
    """one decode configuration of the `configs` object: timed, priced against the HBM roofline, its first tokens
    checked against the CPU port's, the CPU port timed on the same kind of step"""
    d = Decode(lib, model_name, kind, weights, prompt)
    wall, positions = d.timed(steps, warmup)
    step_us, step_bytes = d.events(steps, warmup)
    gbs = step_bytes / (step_us * 1e-6) / 1e9
    res = {"workload": name, "ms_per_step": wall * 1e3 / steps, "tokens_per_s": steps / wall, "steps": steps,
           "positions": f"{min(positions)}..{max(positions)}",
           "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                        "bytes_per_launch": step_bytes, "us_per_launch": step_us, "traffic": None}}
    if cpu_seconds > 0:
        cp = prompt if cpu_prompt is None else cpu_prompt
        rate, cpu_toks, sample = cpu_decode(d.cfg, dequantised(weights, kind, d.llama), cp, cpu_seconds, d.llama, cpu_steps)
        d.prompt = cp
        got = d.first_tokens(len(cpu_toks))
        if got != cpu_toks:
            raise SystemExit(f"bench: {name}: tokens {got} differ from the CPU port's {cpu_toks}; no figure is reported for a wrong result")
        res["checked"] = f"{len(cpu_toks)} greedy tokens equal the CPU port's"
        res["cpu_baseline"] = {"value": rate, "unit": "tokens/s", "cores": 1, "kind": "port", "sample": sample}
    d.close()
    return res


def byoc_decode(cfg, weights, prompt, steps, want_tokens):
    """the plug-in path: the compiled graph's node list, every item through cthip_program_launch; walked inside the
    library (one call per forward), and -- fewer steps, for comparison -- node by node on the host"""
    from caten_amd import graphs
    from caten_amd.buffer import transfer_into_array

    def run(native, nsteps):
        g = graphs.GPT2Graph(cfg, weights, native=native)
        toks = [int(t) for t in prompt]
        tok = int(np.asarray(transfer_into_array(g.forward(toks, 0))).ravel()[0])
        got, n = [tok], len(toks)
        for _ in range(3):  # warm-up steps (pools of the step's shapes, uploads)
            tok = int(np.asarray(transfer_into_array(g.forward([tok], n))).ravel()[0])
            got.append(tok)
            n += 1
        t0 = time.perf_counter()
        for _ in range(nsteps):
            tok = int(np.asarray(transfer_into_array(g.forward([tok], n))).ravel()[0])
            got.append(tok)
            n += 1
        wall = time.perf_counter() - t0
        routes, launches = g.routes(), g.n_kernels
        g.close()
        k = min(len(got), len(want_tokens))
        if want_tokens and got[:k] != want_tokens[:k]:
            raise SystemExit(f"bench: plug-in path: tokens {got[:k]} differ from the CPU port's {want_tokens[:k]}")
        return wall, routes, launches, k

    wall, routes, launches, k = run(True, steps)
    host_wall = run(False, max(5, steps // 5))[0] / max(5, steps // 5)
    return {"value": steps / wall, "unit": "tokens/s", "ms_per_step": wall * 1e3 / steps, "steps": steps,
            "launches_per_step": launches, "weights": "fp32 (what gguf->state-dict hands a Caten graph whatever the file's type)",
            "what": "GPT-2-small graph as Allocate / scalar / JIT_KERNEL nodes, walked inside the library (cthip_vm_run, one call "
                    "per forward); one cthip_program_launch per Schedule-Item, token returned to the host after every forward "
                    "(the reference's gpt2-generate loop)",
            "ms_per_step_walked_on_the_host": host_wall * 1e3,
            "hand_written_items": sorted(k for k, v in routes.items() if v != "rendered"),
            "rendered_items": sorted(k for k, v in routes.items() if v == "rendered"),
            "checked": f"{k} greedy tokens equal the CPU port's" if want_tokens else "unchecked (no CPU leg)"}


def lm_head_probe(lib, cfg, weights, kind, llama):
    """the largest single launch of a step: final norm -> lm_head GEMV.  "warm": the same matrix back to back -- it
    stays in the 256 MB Infinity Cache; "cold": the launches rotate over enough copies of the matrix (> 256 MB
    together) that every one streams from HBM.  Also the streaming rate this box reaches (a 256 MiB copy)."""
    import ctypes as C
    from caten_amd import _lib, ops
    from caten_amd.llm import Tensor
    V, D = cfg["vocab"], cfg["dim"]
    ms = C.c_float()
    t = Tensor.from_f32(weights["lm_head"], kind)
    wm0 = ops.WeightMatrix(kind, t.raw, V, D)
    ncopies = max(2, int(np.ceil(1.25 * (256 << 20) / wm0.nbytes)))
    wms = [wm0] + [ops.WeightMatrix(kind, t.raw, V, D) for _ in range(ncopies - 1)]
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
    for a in [ca, cb, dx, dg, dy] + ([db] if db else []):
        a.free()
    for w in wms:
        w.free()
    return {"kernel": f"cthip::k_gemv<{kind}> on lm_head ({V}x{D}) with the {'RMSNorm' if llama else 'ln_f'} prologue, the step's largest launch",
            "bytes_per_launch": gemv_bytes, "warm_infinity_cache": lm_warm, "cold_hbm": lm_cold}, copy_gbs


def other_configs(lib, args, gpt2_weights, prompt):
    """the benchmark configurations beside the headline one, each checked, each with its CPU-port sample"""
    import bench_items
    import bench_prefill
    from caten_amd import synth
    cpu = args.cpu_seconds > 0
    out = {}
    items = bench_items.measure(rendered_items=False)
    ci = cpu_items() if cpu else {}
    pick = lambda key: [o for o in items if o["item"].startswith(key)]  # noqa: E731
    mm = pick("relu(matmul)")
    out["C1 relu(matmul) 1024^3 fp32"] = {
        "fp32_mfma": {k: mm[0][k] for k in ("us", "achieved", "unit", "peak", "frac")},
        "routed_default_bf16x3_terms": {k: mm[1][k] for k in ("us", "achieved", "unit", "peak", "frac")},
        "bound": "mfma", "checked": "32 sampled rows against fp64, rtol 1e-3 / atol 1e-4", "cpu_baseline": ci.get("relu(matmul) 1024^3")}
    copy = pick("device-to-device copy")[0]
    for key, nm, ck in (("LayerNorm->softmax fused", "C2a LayerNorm->softmax (64,1024,768) fp32, one kernel", "LayerNorm->softmax (64,1024,768)"),
                        ("GELU(tanh)", "C2b GELU(tanh) (64,1024,768) fp32", "GELU(tanh) (64,1024,768)")):
        o = pick(key)[0]
        out[nm] = {"us": o["us"], "bound": "hbm", "achieved": o["achieved"], "unit": "GB/s", "peak": 8000.0, "frac": o["frac"],
                   "frac_of_copy": o["frac_of_copy"], "bytes_per_launch": o["bytes"], "measured_copy_GBs": copy["achieved"],
                   "checked": "64 sampled rows against fp64, rtol 1e-3 / atol 1e-5", "cpu_baseline": ci.get(ck)}
    cfg = synth.GPT2_CONFIGS["gpt2"]
    out["C3 GPT-2-small fp32 decode"] = decode_config(
        lib, "GPT-2-small shape, fp32 weights, fp32 KV, 16-token prompt, 100-token greedy decode", "gpt2", "f32", gpt2_weights, prompt,
        100, 5, min(args.cpu_seconds, 6.0), cpu_steps=24)
    pf = bench_prefill.measure("gpt2", "q8_0", 512, modes=(0, 2), weights=gpt2_weights, reps=5)
    out["C4 GPT-2-small Q8_0 prefill, 512 tokens"] = {
        "ms": pf[1]["ms"], "tokens_per_s": pf[1]["tokens_per_s"], "bound": "mfma", "achieved": pf[1]["linear_TFLOPs"], "unit": "TFLOP/s",
        "peak": 2500.0, "frac": pf[1]["frac"], "operands": "activations as two bf16 terms, Q8_0 integers exact in bf16, fp32 accumulation",
        "fp32_operands": {"ms": pf[0]["ms"], "achieved": pf[0]["linear_TFLOPs"], "peak": 157.3, "frac": pf[0]["frac"]},
        "linear_GFLOP": pf[1]["linear_GFLOP"], "attention_GFLOP": pf[1]["attention_GFLOP"],
        "checked": "logits against the fp32-operand run, rtol 1e-3 / atol 1e-4, same greedy token"}
    if cpu:
        # the CPU port on a bounded sample of the prompt: 8 of the 512 rows through one forward
        import oracle
        m = oracle.GPT2(cfg, dequantised(gpt2_weights, "q8_0", False))
        rows = synth.prompt(cfg["vocab"], 8, seed=0)
        t0 = time.perf_counter()
        m.forward([float(t) for t in rows], 0, onehot=True, all_logits=True)
        el = time.perf_counter() - t0
        out["C4 GPT-2-small Q8_0 prefill, 512 tokens"]["cpu_baseline"] = {
            "value": 8 / el, "unit": "tokens/s", "cores": 1, "kind": "port", "sample": f"an 8-token prompt (of 512), fp32 dequantised weights, {el:.1f} s"}
    # Llama-1.1B shape, Q4_0
    lcfg = synth.LLAMA_CONFIGS["llama-1.1b"]
    lw = synth.llama_weights(lcfg, seed=0, threads=THREADS)
    lprompt = synth.prompt(lcfg["vocab"], 128, seed=0)
    out["C5 Llama-1.1B-shape Q4_0 decode"] = decode_config(
        lib, "Llama-1.1B shape (22L d2048 32q/4kv heads, SwiGLU 5632, RoPE), Q4_0 weights, 128-token prompt (one batch), 128-token greedy decode",
        "llama-1.1b", "q4_0", lw, lprompt, 128, 4, min(args.cpu_seconds, 12.0), cpu_prompt=lprompt[:1], cpu_steps=3)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--model", default="gpt2")
    ap.add_argument("--kind", default="q8_0")
    ap.add_argument("--prompt", type=int, default=16)
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="CPU baseline budget of the headline workload (0 disables every CPU leg)")
    ap.add_argument("--configs", default="all", choices=("all", "headline"),
                    help="all: the other benchmark configurations and the plug-in path are measured in the same run")
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

    from caten_amd import _lib, synth, ops
    llama = args.model in synth.LLAMA_CONFIGS
    cfg = dict(synth.LLAMA_CONFIGS[args.model] if llama else synth.GPT2_CONFIGS[args.model])
    weights = synth.llama_weights(cfg, seed=0, threads=THREADS) if llama else synth.gpt2_weights(cfg, seed=0)
    prompt = synth.prompt(cfg["vocab"], args.prompt, seed=0)
    lib = _lib.init(0)
    if args.no_graph:
        _lib.check(lib.cthip_set_option(b"decoder_graph", 0))
    for kv in args.option:
        name, value = kv.split("=")
        _lib.check(lib.cthip_set_option(name.encode(), int(value)))

    # ---- the headline workload: exactly K decode steps timed on the host clock, then again under HIP events ----
    d = Decode(lib, args.model, args.kind, weights, prompt)
    wall, positions = d.timed(args.steps, args.warmup)
    ms_per_step = wall * 1e3 / args.steps
    tok_s = args.steps / wall
    step_us, step_bytes = d.events(args.steps, args.warmup)
    step_gbs = step_bytes / (step_us * 1e-6) / 1e9
    lm_head, copy_gbs = lm_head_probe(lib, cfg, weights, args.kind, llama)
    traffic, traffic_positions = profile_traffic(args.model, args.kind)

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
                     "traffic_from": None if traffic is None else
                     f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE over the step's dispatches at positions {traffic_positions} "
                     f"(profiles/decode_{args.model}_{args.kind}_step_pmc.txt), not re-counted by this run",
                     "measured_copy": {"achieved": copy_gbs, "unit": "GB/s", "frac": copy_gbs / HBM_PEAK_GBS,
                                       "what": "256 MiB device-to-device copy on the library's stream, bytes read + written"},
                     "kernel": "one decode step = one replay of the step's launches (the dequant-in-register Linear "
                               "kernels, attention, argmax), packed weights + norms / biases + embedding rows + KV rows",
                     "bytes_per_launch": step_bytes, "us_per_launch": step_us,
                     "lm_head": lm_head},
    }
    if args.calibrate_copy:
        n = 256 << 20
        a, b = ops.DeviceArray((n,), np.uint8), ops.DeviceArray((n,), np.uint8)
        _lib.check(lib.cthip_d2d(b.ptr, a.ptr, n))
        _lib.check(lib.cthip_sync())
    cpu_toks = []
    if args.cpu_seconds > 0:
        rate, cpu_toks, sample = cpu_decode(cfg, dequantised(weights, args.kind, llama), prompt, args.cpu_seconds, llama)
        got = d.first_tokens(len(cpu_toks))
        if got != cpu_toks:
            raise SystemExit(f"bench: tokens {got} differ from the CPU port's {cpu_toks}; no figure is reported for a wrong result")
        res["checked"] = f"{len(cpu_toks)} greedy tokens equal the CPU port's"
        res["cpu_baseline"] = {"value": rate, "unit": "tokens/s", "cores": 1, "kind": "port", "sample": sample}
    d.close()
    if args.configs == "all" and not llama and args.model == "gpt2":
        res["configs"] = other_configs(lib, args, weights, prompt)
        if "cpu_baseline" in res:
            res["cpu_baseline"]["items"] = {k: v.get("cpu_baseline") for k, v in res["configs"].items()}
        # the plug-in path on the fp32 graph; its tokens against the fp32 CPU port's (the C3 leg's check is on the same weights)
        want = []
        if args.cpu_seconds > 0:
            _, want, _ = cpu_decode(cfg, weights, prompt, 1.0, False, max_steps=12)
        res["byoc_path"] = byoc_decode(cfg, weights, prompt, 50, want)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
